"""Every statement the gfx950 emitter lowers, on values: the programs of tests/dsl_op_programs.py run
on the GPU and each block of their output is compared with the same operation computed on the CPU in
float32 (float64 for the products).  Bars: exact for data movement, masks, layout changes, comparisons,
min/max and the bf16 round trip; a few ulp (rtol 2e-5) for arithmetic and transcendental functions,
whose GPU versions are the fast hardware instructions."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
T = 64


@pytest.fixture(scope="module")
def rt():
    from tests import dsl_op_programs as op_programs
    from tyr_amd.dsl import runtime
    return op_programs, runtime, op_programs.load()


def close(got, want, exact=False):
    got, want = got.cpu(), want.cpu()
    if exact:
        assert torch.equal(torch.nan_to_num(got, nan=1234.5), torch.nan_to_num(want, nan=1234.5))
    else:
        assert torch.allclose(got, want, rtol=2e-5, atol=2e-6, equal_nan=True), float((got - want).abs().nan_to_num().max())


def test_unary(rt):
    P, runtime, L = rt
    from tyr_amd.dsl.ir import UNARY_OPS
    g = torch.Generator().manual_seed(1)
    x = torch.rand(T, T, generator=g) * 1.9 + 0.1
    out = torch.full((2 * len(UNARY_OPS) * T, T), 77.0).cuda()
    runtime.launch(P.dslOpsUnary(), [x.cuda(), out], library=L)
    torch.cuda.synchronize()
    F = torch.nn.functional
    ref = {"Exp": torch.exp, "Exp2": torch.exp2, "Log": torch.log, "Log2": torch.log2, "Abs": torch.abs,
           "Relu": torch.relu, "Copy": lambda v: v, "Neg": torch.neg, "Sqrt": torch.sqrt, "Rsqrt": torch.rsqrt,
           "Tanh": torch.tanh, "FastTanh": torch.tanh, "Sigmoid": torch.sigmoid,
           "Gelu": lambda v: F.gelu(v, approximate="tanh"), "Silu": F.silu, "Swish": F.silu, "Sin": torch.sin,
           "Cos": torch.cos, "Recip": torch.reciprocal, "Square": torch.square, "Zero": torch.zeros_like,
           "One": torch.ones_like, "PosInfty": lambda v: torch.full_like(v, float("inf")),
           "NegInfty": lambda v: torch.full_like(v, float("-inf"))}
    exact = {"Abs", "Relu", "Copy", "Neg", "Zero", "One", "PosInfty", "NegInfty", "Square"}
    for half, src in enumerate((x, x - 1.0)):
        for i, op in enumerate(UNARY_OPS):
            b = half * len(UNARY_OPS) + i
            close(out[b * T:(b + 1) * T], ref[op](src), exact=op in exact)


def test_binary_broadcast_reduce_and_vectors(rt):
    P, runtime, L = rt
    g = torch.Generator().manual_seed(2)
    x = torch.rand(T, T, generator=g) + 0.5
    y = torch.rand(T, T, generator=g) + 0.5
    vr = torch.rand(T, generator=g) + 0.5
    vc = torch.rand(T, generator=g) + 0.5
    out = torch.full((len(P.BINARY_BLOCKS) * T, T), 77.0).cuda()
    vout = torch.full((len(P.VECTOR_BLOCKS) * T,), 77.0).cuda()
    runtime.launch(P.dslOpsBinary(), [x.cuda(), y.cuda(), vr.cuda(), vc.cuda(), out, vout], library=L)
    torch.cuda.synchronize()
    R, C = vr[None, :], vc[:, None]
    want = {"add": x + y, "sub": x - y, "mul": x * y, "div": x / y, "max": torch.maximum(x, y), "min": torch.minimum(x, y),
            "scalarMul": x * 2.5, "scalarAdd": x - 0.75, "fma": x * y + x, "addRow": x + R, "subRow": x - R,
            "mulRow": x * R, "divRow": x / R, "addCol": x + C, "subCol": x - C, "mulCol": x * C, "divCol": x / C,
            "broadcastRow": R.expand(T, T), "broadcastCol": C.expand(T, T), "outer": torch.outer(vc, vr)}
    exact = {"add", "sub", "mul", "max", "min", "scalarMul", "scalarAdd", "addRow", "subRow", "mulRow", "addCol",
             "subCol", "mulCol", "broadcastRow", "broadcastCol", "outer"}
    for i, name in enumerate(P.BINARY_BLOCKS):
        close(out[i * T:(i + 1) * T], want[name], exact=name in exact)
    wantv = {"rowMax": x.max(1).values, "rowMin": x.min(1).values, "rowSum": x.sum(1), "rowProd": x.double().prod(1).float(),
             "colMax": x.max(0).values, "colMin": x.min(0).values, "colSum": x.sum(0), "colProd": x.double().prod(0).float(),
             "rowMaxAccum": torch.maximum(x.max(1).values, vc), "rowSumAccum": x.sum(1) + vc, "addVec": vc + vc + vc,
             "mulVec": vr * vr, "expVec": torch.exp(vr), "scalarMulVec": vc * -3.0,
             "iota": 2.0 + 0.5 * torch.arange(T, dtype=torch.float32), "fill": torch.full((T,), 7.25),
             "convertVec": vr.bfloat16().float()}
    exactv = {"rowMax", "rowMin", "colMax", "colMin", "rowMaxAccum", "addVec", "mulVec", "scalarMulVec", "iota", "fill",
              "convertVec"}
    for i, name in enumerate(P.VECTOR_BLOCKS):
        got = vout[i * T:(i + 1) * T].cpu()
        if name in exactv:
            assert torch.equal(got, wantv[name]), name
        else:                                    # sums and products: order of accumulation differs
            assert torch.allclose(got, wantv[name], rtol=1e-5, atol=1e-5), name


def test_masks(rt):
    P, runtime, L = rt
    g = torch.Generator().manual_seed(3)
    x = torch.rand(T, T, generator=g) + 1.0
    out = torch.full((len(P.MASK_BLOCKS) * T, T), 77.0).cuda()
    runtime.launch(P.dslOpsMasks(), [x.cuda(), out], library=L)
    torch.cuda.synchronize()
    i, j = torch.meshgrid(torch.arange(T), torch.arange(T), indexing="ij")
    keep = {"makeCausal": lambda: j <= i, "makeCausalT": lambda: j >= i, "tril": lambda d: j <= i + d,
            "triu": lambda d: j >= i + d, "rightFill": lambda c: j < c, "leftFill": lambda c: j >= c,
            "upperFill": lambda r: i >= r, "lowerFill": lambda r: i < r,
            "upperRightFill": lambda r, c: ~((i < r) & (j >= c))}
    for b, (name, args, fill) in enumerate(P.MASK_BLOCKS):
        want = torch.where(keep[name](*args), x, torch.tensor(0.0 if fill is None else fill))
        close(out[b * T:(b + 1) * T], want, exact=True)
    # tril / triu agree with the library routines of the same name
    close(out[4 * T:5 * T], torch.tril(x), exact=True)
    close(out[7 * T:8 * T], torch.triu(x, 4), exact=True)


def test_layout_changes(rt):
    P, runtime, L = rt
    g = torch.Generator().manual_seed(4)
    x = torch.rand(T, T, generator=g)
    out = torch.full((len(P.LAYOUT_BLOCKS) * T, T), 77.0).cuda()
    runtime.launch(P.dslOpsLayout(), [x.cuda(), out], library=L)
    torch.cuda.synchronize()
    blk = lambda n: out[n * T:(n + 1) * T]
    close(blk(0), x.t(), exact=True)
    close(blk(1), x, exact=True)
    close(blk(2), x, exact=True)
    close(blk(3), torch.cat([x[:, 32:], x[:, :32]], 1), exact=True)
    close(blk(4), x.bfloat16().float(), exact=True)
    close(blk(5), torch.cat([x[32:], torch.zeros(32, T)], 0), exact=True)


def test_products(rt):
    P, runtime, L = rt
    M, N, K = 64, 96, 32
    torch.manual_seed(5)
    a_mk, a_km = torch.randn(M, K).bfloat16(), torch.randn(K, M).bfloat16()
    b_kn, b_nk = torch.randn(K, N).bfloat16(), torch.randn(N, K).bfloat16()
    c = torch.randn(M, N)
    out = torch.full((5 * M, N), 77.0).cuda()
    runtime.launch(P.dslOpsMma(), [a_mk.cuda(), a_km.cuda(), b_kn.cuda(), b_nk.cuda(), c.cuda(), out], library=L)
    torch.cuda.synchronize()
    d = lambda t: t.double()
    want = [d(a_mk) @ d(b_kn) + d(c), d(a_mk) @ d(b_nk).t() + d(c), d(a_km).t() @ d(b_kn) + d(c),
            d(a_km).t() @ d(b_nk).t() + d(c), d(a_mk) @ d(b_kn)]
    for i, w in enumerate(want):
        got = out[i * M:(i + 1) * M].cpu().double()
        assert float((got - w).norm() / w.norm()) <= 1e-6, i
        assert float((got - w).abs().max()) <= 1e-4, i


@pytest.mark.parametrize("n", [1, 3])
def test_control_flow_and_scalars(rt, n):
    P, runtime, L = rt
    g = torch.Generator().manual_seed(6)
    x = torch.rand(3 * T, 2 * T, generator=g)
    s = torch.tensor([1.5, 0, 0, 0, 0, 99.0]).cuda()
    out = torch.full((T, 2 * T), 77.0).cuda()
    runtime.launch(P.dslOpsControl(), [x.cuda(), s, out, n], grid=(2, 1, 1), library=L)
    torch.cuda.synchronize()
    acc = sum(x[i * T:(i + 1) * T] for i in range(n))
    assert torch.allclose(out[:, :T].cpu(), acc[:, :T], rtol=1e-6, atol=1e-6)
    assert torch.allclose(out[:, T:].cpu(), 2.0 * acc[:, T:], rtol=1e-6, atol=1e-6)
    assert s.cpu().tolist() == [1.5, 3.0, -(1.5 * 3.0 + 1.0), float(max(n, 5) % 4), 1.5 if n >= 2 else 0.0, 42.0]


@pytest.mark.parametrize("block", [32, 128])
def test_scans_and_atomic_accumulation(rt, block):
    P, runtime, L = rt
    g = torch.Generator().manual_seed(8)
    x = torch.rand(T, T, generator=g) * 0.2 + 0.9
    out = torch.full((len(P.SCAN_BLOCKS) * T, T), 77.0).cuda()
    acc0 = torch.rand(T, T, generator=g)
    vacc0 = torch.rand(2 * T, generator=g)
    acc, vacc = acc0.cuda(), vacc0.cuda()
    runtime.launch(P.dslOpsScanAtomic(), [x.cuda(), out, acc, vacc], block=(block, 1, 1), library=L)
    torch.cuda.synchronize()
    xd = x.double()
    want = {"cumsumRow": xd.cumsum(1), "cumsumCol": xd.cumsum(0), "cumprodRow": xd.cumprod(1), "cumprodCol": xd.cumprod(0)}
    for i, name in enumerate(P.SCAN_BLOCKS):
        got = out[i * T:(i + 1) * T].cpu().double()
        assert torch.allclose(got, want[name], rtol=1e-5, atol=1e-5), name
    waves = block // 32                                      # every wave of the workgroup adds
    assert torch.allclose(acc.cpu(), acc0 + waves * x, rtol=1e-6, atol=1e-6)
    rs = x.sum(1)
    assert torch.allclose(vacc.cpu(), vacc0 + waves * torch.cat([rs, rs]), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("block", [32, 128])
def test_full_axis_fma_tags_and_in_place_transpose(rt, block):
    P, runtime, L = rt
    g = torch.Generator().manual_seed(9)
    x, y, z = (torch.rand(T, T, generator=g) * 0.5 + 0.75 for _ in range(3))
    v = torch.rand(T, generator=g) * 0.1 + 0.95
    out = torch.full((len(P.FULL_TILE_BLOCKS) * T, T), 77.0).cuda()
    vout = torch.full((len(P.FULL_VECTOR_BLOCKS) * T,), 77.0).cuda()
    runtime.launch(P.dslOpsFull(), [x.cuda(), y.cuda(), z.cuda(), v.cuda(), out, vout], block=(block, 1, 1), library=L)
    torch.cuda.synchronize()
    xd, yd, zd, vd = x.double(), y.double(), z.double(), v.double()
    want_t = {"fmaAxBtC": xd * yd + zd, "fmaAxCtB": xd * zd + yd, "transposeInPlace": xd.T}
    for i, name in enumerate(P.FULL_TILE_BLOCKS):
        got = out[i * T:(i + 1) * T].cpu().double()
        assert torch.allclose(got, want_t[name], rtol=1e-6, atol=1e-6), name
    ones = torch.ones(T, dtype=torch.float64)
    want_v = {"fullMaxOfVec": vd.max() * ones, "fullSumOfVec": vd.sum() * ones, "fullMinOfTile": xd.min() * ones,
              "fullSumOfTile": xd.sum() * ones, "fullSumAccum": vd.sum() + vd, "fullCumsum": vd.cumsum(0),
              "fullCumprod": vd.cumprod(0), "fullSumOfColVec": xd.sum() * ones}
    for i, name in enumerate(P.FULL_VECTOR_BLOCKS):
        got = vout[i * T:(i + 1) * T].cpu().double()
        assert torch.allclose(got, want_v[name], rtol=2e-5, atol=1e-5), (name, got[:4], want_v[name][:4])
