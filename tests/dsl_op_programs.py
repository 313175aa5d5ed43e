"""Small tile programs that put every statement the gfx950 emitter lowers through the whole path
(builder -> emitter -> hipcc -> GPU), one family of statements per program.  They are test programs, not part
of the product: `build()` below compiles them into `tests/build/libtyr_dsl_ops.so` and they exist for the parity tests: each writes the
result of every operation it covers to its own block of the output, where the test compares it with
the same operation done by the CPU checker.  The reference tests its lowering one statement at a time
on text (Tyr/GPU/Codegen/Tests.lean:31-431); these do it on values."""
from __future__ import annotations

from tyr_amd.dsl.builder import KernelBuilder
from tyr_amd.dsl.ir import UNARY_OPS, Kernel

T = 64


def _emit_tile(k, out, stage, tile, row_block, cols_block=None):
    """registers -> LDS -> block `row_block` of `out`.  The waves of a workgroup all run the whole
    program, so the staging tile is fenced by barriers like any LDS tile that is reused."""
    k.sync()
    k.store(stage, tile)
    z = k.constIntVal(0)
    r = k.constIntVal(row_block)
    c = z if cols_block is None else k.constIntVal(cols_block)
    from tyr_amd.dsl.builder import RTileCoord
    k.storeGlobal(out, stage, RTileCoord(z, z, r, c))


def dslOpsUnary() -> Kernel:
    """out block i = UNARY_OPS[i] applied to x (blocks 0..23) and to x - 1 (blocks 24..47)."""
    k = KernelBuilder("dslOpsUnary")
    x_ptr = k.gptr("Float32", "x")
    out = k.gptr("Float32", "out")
    coord = k.blockCoord2D()
    xs = k.allocST("Float32", T, T)
    stage = k.allocST("Float32", T, T)
    x = k.allocRT("Float32", T, T)
    xm = k.allocRT("Float32", T, T)
    y = k.allocRT("Float32", T, T)
    k.loadGlobal(xs, x_ptr, coord)
    k.load(x, xs)
    k.scalarAdd(xm, x, -1.0)
    for half, src in enumerate((x, xm)):
        for i, op in enumerate(UNARY_OPS):
            k.unaryOp(op, y, src)
            _emit_tile(k, out, stage, y, half * len(UNARY_OPS) + i)
    return k.build()


BINARY_BLOCKS = ("add", "sub", "mul", "div", "max", "min", "scalarMul", "scalarAdd", "fma", "addRow", "subRow", "mulRow",
                 "divRow", "addCol", "subCol", "mulCol", "divCol", "broadcastRow", "broadcastCol", "outer")
VECTOR_BLOCKS = ("rowMax", "rowMin", "rowSum", "rowProd", "colMax", "colMin", "colSum", "colProd", "rowMaxAccum",
                 "rowSumAccum", "addVec", "mulVec", "expVec", "scalarMulVec", "iota", "fill", "convertVec")


def dslOpsBinary() -> Kernel:
    """x, y 64x64 f32; vr (used along rows) and vc (used down columns) 64 f32.  Tile results go to
    `out` in the order of BINARY_BLOCKS, vector results to `vout` in the order of VECTOR_BLOCKS."""
    k = KernelBuilder("dslOpsBinary")
    x_ptr = k.gptr("Float32", "x")
    y_ptr = k.gptr("Float32", "y")
    vr_ptr = k.gptr("Float32", "vr")
    vc_ptr = k.gptr("Float32", "vc")
    out = k.gptr("Float32", "out")
    vout = k.gptr("Float32", "vout")
    coord = k.blockCoord2D()
    xs = k.allocST("Float32", T, T)
    ys = k.allocST("Float32", T, T)
    stage = k.allocST("Float32", T, T)
    vs = k.allocSV("Float32", T)
    x = k.allocRT("Float32", T, T)
    y = k.allocRT("Float32", T, T)
    t = k.allocRT("Float32", T, T)
    vr = k.allocRV("Float32", T)
    vc = k.allocRV("Float32", T)
    k.loadGlobal(xs, x_ptr, coord)
    k.loadGlobal(ys, y_ptr, coord)
    k.load(x, xs)
    k.load(y, ys)
    k.loadVecGlobalRow(vs, vr_ptr, coord)
    k.loadVec(vr, vs)
    k.sync()
    k.loadVecGlobal(vs, vc_ptr, coord)                       # the 4-D coordinate form; (0, 0, 0, 0) here
    k.loadVec(vc, vs)

    n = [0]

    def put(tile):
        _emit_tile(k, out, stage, tile, n[0])
        n[0] += 1

    for name in ("add", "sub", "mul", "div", "max", "min"):
        getattr(k, name)(t, x, y); put(t)
    k.scalarMul(t, x, 2.5); put(t)
    k.scalarAdd(t, x, -0.75); put(t)
    k.fma(t, x, y, x); put(t)
    for name in ("addRow", "subRow", "mulRow", "divRow"):
        getattr(k, name)(t, x, vr); put(t)
    for name in ("addCol", "subCol", "mulCol", "divCol"):
        getattr(k, name)(t, x, vc); put(t)
    k.broadcastRow(t, vr); put(t)
    k.broadcastCol(t, vc); put(t)
    k.outer(t, vc, vr); put(t)
    assert n[0] == len(BINARY_BLOCKS)

    m = [0]

    def putv(vec):
        k.sync()
        k.storeVec(vs, vec)
        if m[0] % 2:
            k.storeVecGlobalRow(vout, vs, k.rowCoord(k.constIntVal(m[0])))
        else:                                                # 4-D form: vector m[0] of row 0
            k.storeVecGlobal(vout, vs, coord.withCol(k.constIntVal(m[0])))
        m[0] += 1

    for name in ("rowMax", "rowMin", "rowSum", "rowProd", "colMax", "colMin", "colSum", "colProd"):
        v = k.allocRV("Float32", T)
        getattr(k, name)(v, x); putv(v)
    v = k.allocRV("Float32", T); k.rowMaxAccum(v, x, vc); putv(v)
    v = k.allocRV("Float32", T); k.rowSumAccum(v, x, vc); putv(v)
    v = k.allocRV("Float32", T); k.addVec(v, vc, vc); k.addVec(v, v, vc); putv(v)          # 3 vc
    v = k.allocRV("Float32", T); k.mulVec(v, vr, vr); putv(v)
    v = k.allocRV("Float32", T); k.expVec(v, vr); putv(v)
    v = k.allocRV("Float32", T); k.scalarMulVec(v, vc, -3.0); putv(v)
    v = k.allocRV("Float32", T); k.iotaVec(v, 2.0, 0.5); putv(v)
    v = k.allocRV("Float32", T); k.fillVecScalar(v, k.constFloatVal(7.25)); putv(v)
    vb = k.allocRV("BFloat16", T); k.convertVec(vb, vr)
    v = k.allocRV("Float32", T); k.convertVec(v, vb); putv(v)
    assert m[0] == len(VECTOR_BLOCKS)
    return k.build()


MASK_BLOCKS = (("makeCausal", (), None), ("makeCausal", (), -5.0), ("makeCausalT", (), 1.5), ("tril", (-3,), -1.0),
               ("tril", (0,), None), ("tril", (5,), 9.0), ("triu", (-2,), 3.0), ("triu", (4,), None),
               ("rightFill", (20,), -2.0), ("leftFill", (7,), 4.0), ("upperFill", (9,), 6.0), ("lowerFill", (50,), -7.0),
               ("upperRightFill", (33, 10), 8.0))


def dslOpsMasks() -> Kernel:
    k = KernelBuilder("dslOpsMasks")
    x_ptr = k.gptr("Float32", "x")
    out = k.gptr("Float32", "out")
    coord = k.blockCoord2D()
    xs = k.allocST("Float32", T, T)
    stage = k.allocST("Float32", T, T)
    x = k.allocRT("Float32", T, T)
    y = k.allocRT("Float32", T, T)
    k.loadGlobal(xs, x_ptr, coord)
    k.load(x, xs)
    for i, (name, args, fill) in enumerate(MASK_BLOCKS):
        getattr(k, name)(y, x, *args, fill)
        _emit_tile(k, out, stage, y, i)
    return k.build()


LAYOUT_BLOCKS = ("transpose", "swapLayout", "transposeBack", "swapHalves", "bf16RoundTrip", "sliceRows")


def dslOpsLayout() -> Kernel:
    """x 64x64 f32 -> x^T (through a Col tile), x (layout swapped to Col and stored), x (transposed
    twice), [x right half | x left half], bf16-rounded x, and rows 32..63 of x over rows 0..31."""
    k = KernelBuilder("dslOpsLayout")
    x_ptr = k.gptr("Float32", "x")
    out = k.gptr("Float32", "out")
    coord = k.blockCoord2D()
    xs = k.allocST("Float32", T, T)
    stage = k.allocST("Float32", T, T)
    half_stage = k.allocST("Float32", 32, T)
    x = k.allocRT("Float32", T, T)
    xt = k.allocRT("Float32", T, T, "Col")
    xc = k.allocRT("Float32", T, T, "Col")
    back = k.allocRT("Float32", T, T)
    k.loadGlobal(xs, x_ptr, coord)
    k.load(x, xs)
    k.transpose(xt, x)
    _emit_tile(k, out, stage, xt, 0)
    k.swapLayout(xc, x)
    _emit_tile(k, out, stage, xc, 1)
    k.transpose(back, xt)
    _emit_tile(k, out, stage, back, 2)
    left = k.allocRT("Float32", T, 32)
    right = k.allocRT("Float32", T, 32)
    k.sliceCols(left, x, 0, 32)
    k.sliceCols(right, x, 32, 32)
    k.concatCols(back, right, left)
    _emit_tile(k, out, stage, back, 3)
    xb = k.allocRT("BFloat16", T, T)
    k.convert(xb, x)
    k.convert(back, xb)
    _emit_tile(k, out, stage, back, 4)
    lower = k.allocRT("Float32", 32, T)
    k.sliceRows(lower, x, 32, 32)
    k.zero(back)
    _emit_tile(k, out, stage, back, 5)                       # block 5 = zeros ...
    _emit_tile(k, out, half_stage, lower, 10)                # ... with its first 32 rows overwritten (32-row units)
    return k.build()


def dslOpsMma() -> Kernel:
    """The four operand arrangements of the product, M=64, N=96, K=32, plus `mm`:
    out blocks: a_mk b_kn + c | a_mk b_nk^T + c | a_km^T b_kn + c | a_km^T b_nk^T + c | a_mk b_kn."""
    M, N, K = 64, 96, 32
    k = KernelBuilder("dslOpsMma")
    a_mk_p = k.gptr("BFloat16", "a_mk")
    a_km_p = k.gptr("BFloat16", "a_km")
    b_kn_p = k.gptr("BFloat16", "b_kn")
    b_nk_p = k.gptr("BFloat16", "b_nk")
    c_p = k.gptr("Float32", "c")
    out = k.gptr("Float32", "out")
    coord = k.blockCoord2D()
    s_mk = k.allocST("BFloat16", M, K)
    s_km = k.allocST("BFloat16", K, M)
    s_kn = k.allocST("BFloat16", K, N)
    s_nk = k.allocST("BFloat16", N, K)
    s_c = k.allocST("Float32", M, N)
    k.loadGlobal(s_mk, a_mk_p, coord)
    k.loadGlobal(s_km, a_km_p, coord)
    k.loadGlobal(s_kn, b_kn_p, coord)
    k.loadGlobal(s_nk, b_nk_p, coord)
    k.loadGlobal(s_c, c_p, coord)
    a_mk = k.allocRT("BFloat16", M, K)
    a_km = k.allocRT("BFloat16", K, M, "Col")
    b_kn = k.allocRT("BFloat16", K, N, "Col")
    b_nk = k.allocRT("BFloat16", N, K)
    c = k.allocRT("Float32", M, N)
    d = k.allocRT("Float32", M, N)
    k.load(a_mk, s_mk)
    k.load(a_km, s_km)
    k.load(b_kn, s_kn)
    k.load(b_nk, s_nk)
    k.load(c, s_c)
    k.mma(d, a_mk, b_kn, c); _emit_tile(k, out, s_c, d, 0)
    k.mmaT(d, a_mk, b_nk, c); _emit_tile(k, out, s_c, d, 1)
    k.mmaAtB(d, a_km, b_kn, c); _emit_tile(k, out, s_c, d, 2)
    k.mmaAtBt(d, a_km, b_nk, c); _emit_tile(k, out, s_c, d, 3)
    k.mm(d, a_mk, b_kn); _emit_tile(k, out, s_c, d, 4)
    return k.build()


def dslOpsControl() -> Kernel:
    """Runtime loop bound, conditionals and scalar arithmetic.  Workgroup (bx, 0):
    acc = sum over i < n of row tile i of x (column tile bx); it is stored scaled by 2 where bx is odd.
    Thread-independent scalars: s[1] = rows(x) / 64 ; s[2] = -(s[0] * 3 + 1) ; s[3] = max(n, 5) mod 4 ;
    s[4] = s[0] if n >= 2 else 0 ; s[5] = 42 (raw statement, thread 0)."""
    k = KernelBuilder("dslOpsControl")
    x_ptr = k.gptr("Float32", "x")
    s_ptr = k.gptr("Float32", "s")
    out = k.gptr("Float32", "out")
    n = k.kval("UInt32", "n")
    coord = k.blockCoord2D()
    xs = k.allocST("Float32", T, T)
    stage = k.allocST("Float32", T, T)
    acc = k.zeroRT("Float32", T, T)
    t = k.allocRT("Float32", T, T)
    with k.kvrange(0, n) as i:
        k.sync()
        k.loadGlobal(xs, x_ptr, coord.withRow(i.id))
        k.load(t, xs)
        k.add(acc, acc, t)
    one = k.constIntVal(1)
    two = k.constIntVal(2)
    odd = k.scalarCompare("Eq", k.scalarBinary("Mod", coord.c, two), one)
    with k.ifThen(odd):
        k.scalarMul(acc, acc, 2.0)
    with k.orElse():
        k.comment("even column tiles keep the plain sum")
    k.store(stage, acc)
    k.storeGlobal(out, stage, coord.withRow(k.constIntVal(0)))

    rows = k.layoutRows(x_ptr)
    tiles = k.scalarBinary("Div", rows, k.constIntVal(T))
    k.storeFloat32Scalar(s_ptr, one, tiles)
    s0 = k.loadFloat32Scalar(s_ptr, k.constIntVal(0))
    v = k.scalarBinary("Add", k.scalarBinary("Mul", s0, k.constFloatVal(3.0)), k.constFloatVal(1.0))
    k.storeFloat32Scalar(s_ptr, two, k.scalarUnary("Neg", v))
    mx = k.scalarBinary("Max", n, k.constIntVal(5))
    k.storeFloat32Scalar(s_ptr, k.constIntVal(3), k.scalarBinary("Mod", mx, k.constIntVal(4)))
    ge = k.scalarCompare("Ge", n, two)
    k.storeFloat32Scalar(s_ptr, k.constIntVal(4), k.scalarSelect(ge, s0, k.constFloatVal(0.0)))
    tid = k.getThreadIdxX()
    k.emitRaw(f"if ({tid.ident} == 0) {s_ptr.id.ident}.ptr[5] = 42.0f;  // verbatim backend code")
    return k.build()


SCAN_BLOCKS = ("cumsumRow", "cumsumCol", "cumprodRow", "cumprodCol")


def dslOpsScanAtomic() -> Kernel:
    """Scans of x (blocks of `out` in the order of SCAN_BLOCKS) and atomic accumulation: every wave of
    the workgroup adds x to `acc` and the row sums of x to `vacc[0:64]` (row-offset form) and to
    `vacc[64:128]` (4-D coordinate form)."""
    k = KernelBuilder("dslOpsScanAtomic")
    x_ptr = k.gptr("Float32", "x")
    out = k.gptr("Float32", "out")
    acc = k.gptr("Float32", "acc")
    vacc = k.gptr("Float32", "vacc")
    coord = k.blockCoord2D()
    xs = k.allocST("Float32", T, T)
    stage = k.allocST("Float32", T, T)
    vs = k.allocSV("Float32", T)
    x = k.allocRT("Float32", T, T)
    y = k.allocRT("Float32", T, T)
    k.loadGlobal(xs, x_ptr, coord)
    k.load(x, xs)
    for i, name in enumerate(SCAN_BLOCKS):
        getattr(k, name)(y, x)
        _emit_tile(k, out, stage, y, i)
    k.storeGlobalAdd(acc, xs, coord)
    v = k.allocRV("Float32", T)
    k.rowSum(v, x)
    k.storeVec(vs, v)
    k.storeVecGlobalAddRow(vacc, vs, coord)
    k.storeVecGlobalAdd(vacc, vs, coord.withCol(k.constIntVal(1)))
    return k.build()


FULL_TILE_BLOCKS = ("fmaAxBtC", "fmaAxCtB", "transposeInPlace")
FULL_VECTOR_BLOCKS = ("fullMaxOfVec", "fullSumOfVec", "fullMinOfTile", "fullSumOfTile", "fullSumAccum", "fullCumsum",
                      "fullCumprod", "fullSumOfColVec")


def dslOpsFull() -> Kernel:
    """The IR's "Full" axis (reductions over every element, scans along a vector), the two matrix-style FMA tags and the
    in-place transpose of a square tile.  x, y, z 64x64 f32, v 64 f32.  Tile results go to `out` in the order of
    FULL_TILE_BLOCKS, vector results to `vout` in the order of FULL_VECTOR_BLOCKS (a full reduction leaves its result in
    every element of its destination)."""
    from tyr_amd.dsl.ir import stmt
    from tyr_amd.dsl.builder import RTileCoord
    k = KernelBuilder("dslOpsFull")
    x_ptr = k.gptr("Float32", "x")
    y_ptr = k.gptr("Float32", "y")
    z_ptr = k.gptr("Float32", "z")
    v_ptr = k.gptr("Float32", "v")
    out = k.gptr("Float32", "out")
    vout = k.gptr("Float32", "vout")
    coord = k.blockCoord2D()
    xs, ys, zs = (k.allocST("Float32", T, T) for _ in range(3))
    stage = k.allocST("Float32", T, T)
    vs = k.allocSV("Float32", T)
    x, y, z, w = (k.allocRT("Float32", T, T) for _ in range(4))
    k.loadGlobal(xs, x_ptr, coord)
    k.loadGlobal(ys, y_ptr, coord)
    k.loadGlobal(zs, z_ptr, coord)
    k.loadVecGlobalRow(vs, v_ptr, coord)
    k.sync()
    k.load(x, xs)
    k.load(y, ys)
    k.load(z, zs)
    k.emit(stmt("ternary", "FMAAxBtC", w.id, x.id, y.id, z.id))        # x * y + z
    _emit_tile(k, out, stage, w, 0)
    k.emit(stmt("ternary", "FMAAxCtB", w.id, x.id, y.id, z.id))        # x * z + y
    _emit_tile(k, out, stage, w, 1)
    k.copy(w, x)
    k.transpose(w, w)
    _emit_tile(k, out, stage, w, 2)

    z0 = k.constIntVal(0)

    def put(vec, i):
        k.sync()
        k.storeVec(vs, vec)
        k.storeVecGlobal(vout, vs, RTileCoord(z0, z0, z0, k.constIntVal(i)))

    v = k.allocRV("Float32", T)
    k.loadVec(v, vs)
    r = k.allocRV("Float32", T)
    k.emit(stmt("reduce", "Max", "Full", r.id, v.id))
    put(r, 0)
    k.emit(stmt("reduce", "Sum", "Full", r.id, v.id))
    put(r, 1)
    k.emit(stmt("reduce", "Min", "Full", r.id, x.id))
    put(r, 2)
    k.emit(stmt("reduce", "Sum", "Full", r.id, x.id))
    put(r, 3)
    acc = k.allocRV("Float32", T)
    k.copyVec(acc, v)
    k.emit(stmt("reduceAccum", "Sum", "Full", r.id, v.id, acc.id))     # sum(v) + v[i]
    put(r, 4)
    k.emit(stmt("cumsum", "Full", r.id, v.id))
    put(r, 5)
    k.emit(stmt("cumprod", "Full", r.id, v.id))
    put(r, 6)
    c = k.allocRV("Float32", T)
    k.colSum(c, x)                                                     # a per-column vector (the other register layout)
    k.emit(stmt("reduce", "Sum", "Full", r.id, c.id))
    put(r, 7)
    return k.build()


ALL = (dslOpsScanAtomic, dslOpsUnary, dslOpsBinary, dslOpsMasks, dslOpsLayout, dslOpsMma, dslOpsControl, dslOpsFull)


# ---- build step (run by __graft_entry__.build(); the tests only load what it built)
import os as _os

_HERE = _os.path.dirname(_os.path.abspath(__file__))
SRC_PATH = _os.path.join(_HERE, "build", "tyr_dsl_ops.hip")
LIB_PATH = _os.path.join(_HERE, "build", "libtyr_dsl_ops.so")


def build(lib_path: str = LIB_PATH) -> str:
    """Emits the programs above as one HIP translation unit and compiles it for gfx950."""
    from tyr_amd.dsl import build as dsl_build
    return dsl_build.compile_programs(ALL, SRC_PATH, lib_path)


def load():
    from tyr_amd.dsl import runtime
    return runtime.load(LIB_PATH)


if __name__ == "__main__":
    print(build())
