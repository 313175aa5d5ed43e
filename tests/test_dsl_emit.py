"""The tile DSL on CPU: the IR mirrors the reference's statement set, the builder lowers the
reference's end-to-end kernels to the expected statement sequences, the emitter prints the expected
gfx950 calls (the same style of substring goldens as Tyr/GPU/Codegen/Tests.lean:31-431), register-vector
layouts are inferred, NVIDIA-only statements are refused, and the emitted translation unit compiles
with hipcc for gfx950 (cross-compilation, no GPU)."""
import os
import re
import subprocess

import pytest

from tyr_amd import dsl
from tyr_amd.dsl import build as dsl_build
from tyr_amd.dsl import kernels
from tyr_amd.dsl.ir import KSTMT_FIELDS, VarId, stmt, walk

REFERENCE_KSTMT = """declRT declST declRV declSV declSemaphore declGPtr declKVal load store loadAsync storeAsync storeAdd
storeAddAsync storeMinAsync prefetch tmaExpect tmaLoad tmaStore loadGlobal storeGlobal loadGlobalAsync storeGlobalAsync
storeGlobalAdd layoutDim loadVecGlobal storeVecGlobal storeVecGlobalAdd loadVecGlobalCoord storeVecGlobalCoord
storeVecGlobalAddCoord loadScalarGlobal storeScalarGlobal multimemLoadReduce multimemStore multimemRed mma mm mmaFence
mmaCommitGroup mmaAsyncWait tcgen05Mma cpAsyncLoad tmaLoadAsync unary binary ternary scalarMul scalarAdd broadcast
binaryBroadcast reduce reduceAccum cumsum cumprod outer swapLayout transpose convert mask sliceRows sliceCols concatCols
sync arrive arriveAndWait namedBarrierSync namedBarrierArrive warpGroupIdx electOneSync fenceViewAsyncShared
fenceProxyAsync semaphore forLoop forLoopVal ifStmt ifWarpGroup comment getBlockIdx getThreadIdx constInt constFloat
scalarUnary scalarCompare scalarBinary scalarSelect vecIota vecFillScalar raw""".split()


def test_ir_has_every_reference_constructor():
    # the constructor list of Tyr/GPU/Codegen/IR.lean:50-189, in order
    assert list(KSTMT_FIELDS) == REFERENCE_KSTMT


def test_stmt_checks_constructor_and_arity():
    with pytest.raises(ValueError):
        stmt("loadTile", VarId(0), VarId(1))
    with pytest.raises(ValueError):
        stmt("mma", "AB", VarId(0), VarId(1))
    s = stmt("mma", "ABt", VarId(3), VarId(0), VarId(1), VarId(3))
    assert (s.trans, s.dst, s.a, s.b, s.c) == ("ABt", VarId(3), VarId(0), VarId(1), VarId(3))


def ops(kernel):
    return [s.op for s in walk(kernel.body)]


def test_copy_kernel_lowers_like_the_reference():
    # Kernels/Copy.lean:16-26: comment, blockCoord2D (2 constInt + 2 getBlockIdx), allocRT, allocST, then
    # loadGlobal, load, store, storeGlobal, sync
    k = kernels.copy64x64()
    assert [p.name for p in k.params] == ["input", "output"] and all(p.isPointer for p in k.params)
    assert ops(k) == ["declGPtr", "declGPtr", "comment", "constInt", "constInt", "getBlockIdx", "getBlockIdx",
                      "declRT", "declST", "loadGlobal", "load", "store", "storeGlobal", "sync"]
    by = [s for s in k.body if s.op == "getBlockIdx"]
    assert [s.axis for s in by] == [1, 0]                       # row = blockIdx.y, col = blockIdx.x


def test_online_softmax_macro_expands_to_the_reference_sequence():
    # Macros.lean:121-147: copyVec, rowMaxAccum, subVec, expVec, mulCol, mulVec, subCol, exp, rowSumAccum
    k = kernels.tkFlashAttnFwd2BlockLse()
    loop = next(s for s in k.body if s.op == "forLoop")
    assert (loop.lo, loop.hi) == (0, 2)
    body = list(loop.body)
    i = next(n for n, s in enumerate(body) if s.op == "scalarMul")
    assert body[i].scalar == 0.125
    seq = [(s.op, s.args[0]) for s in body[i + 1:i + 10]]
    assert seq == [("unary", "Copy"), ("reduceAccum", "Max"), ("binary", "Sub"), ("unary", "Exp"),
                   ("binaryBroadcast", "Mul"), ("binary", "Mul"), ("binaryBroadcast", "Sub"), ("unary", "Exp"),
                   ("reduceAccum", "Sum")]
    assert [s.args[0] for s in body if s.op == "mma"] == ["ABt", "AB"]   # mmaT s q k s ; mma o p v o


def test_emitted_text_goldens():
    # statement by statement (the recognition of the online-softmax sequence switched off) ...
    src = dsl.emit_kernel(kernels.tkFlashAttnFwd2BlockLse(), fuse_online_softmax=False)
    for needle in [
        "__global__ __launch_bounds__(256) void tkFlashAttnFwd2BlockLse(gl<bf16> v0, gl<bf16> v1, gl<bf16> v2, "
        "gl<bf16> v3, gl<float> v4, uint64_t v5, uint64_t v6)",
        "rt<bf16, 64, 64, layout::col>",                       # v is a Col tile
        "st<bf16, 64, 64>& v", "st<bf16, 64, 64, 32>& v",                # the V tile (read transposed) has the wider row pad
            "unsigned char tyr_lds_pool[19456];",                             # Q / O tile over the V tile, K tile beside them
        "__shared__ sv<float, 64>",
        "wave::mma_ABt(", "wave::mma_AB(",
        "wave::scalar<op_mul>(", "0.125f);",
        "wave::row_reduce<op_max>(", "wave::row_reduce<op_add>(",
        "wave::col_broadcast<op_mul>(", "wave::col_broadcast<op_sub>(", "wave::col_broadcast<op_div>(",
        "wave::unary<op_neg_infty>(", "wave::unary<op_log>(",
        "for (int v", "wave::sync();",
    ]:
        assert needle in src, needle
    # tile coordinates are scaled by the tile shape, as in EmitNew.lean:249-258
    assert re.search(r"wave::gload\(v\d+_next, v1, coord\{\(int\)v\d+, \(int\)v\d+, \(int\)v\d+ \* 64, \(int\)v\d+ \* 64\}\);", src)
    # the vector store takes the row index as its unit coordinate (GlobalLayout.lean:343-349)
    assert re.search(r"wave::store\(v4, v\d+, \(int\)v\d+\);", src)
    # ... and as emitted by default: the ten statements of `scalarMul` + `onlineSoftmax` (Macros.lean:121-147) become one call
    # that leaves the same values in the same operands
    fused = dsl.emit_kernel(kernels.tkFlashAttnFwd2BlockLse())
    assert re.search(r"wave::online_softmax\(v\d+, v\d+, v\d+, v\d+, v\d+, v\d+, 0\.125f\);", fused)
    for gone in ("wave::scalar<op_mul>(", "wave::row_reduce<op_max>(", "wave::col_broadcast<op_sub>(", "wave::row_reduce<op_add>("):
        assert gone not in fused, gone
    assert "wave::col_broadcast<op_div>(" in fused and "wave::unary<op_log>(" in fused        # finalizeSoftmax, computeLSE stay
    # a sequence that differs in one operand is left alone
    k = dsl.KernelBuilder("almost")
    sc, o = k.zeroRT("Float32", 64, 64), k.zeroRT("Float32", 64, 64)
    st_ = k.allocSoftmaxState("Float32", 64)
    k.onlineSoftmax(sc, o, st_)
    k.copyVec(st_.prevMax, st_.rowMax)
    k.rowMaxAccum(st_.rowMax, sc, st_.rowMax)
    k.subVec(st_.scale, st_.rowMax, st_.prevMax)             # operands swapped
    text = dsl.emit_kernel(k.build())
    assert text.count("wave::online_softmax(") == 1 and "wave::row_reduce<op_max>(" in text


def test_register_vector_layouts_are_inferred():
    # LayerNorm: statistics are reduced along rows and broadcast down columns (align); weight and bias
    # are broadcast along rows (ortho), also through convertVec from their bf16 originals
    k = kernels.tkFusedLayerNormResidual1024()
    lay = dsl.infer_rv_layouts(k)
    decl = [s for s in walk(k.body) if s.op == "declRV"]
    assert len(decl) == 12
    f32 = [s.v for s in decl if s.dtype == "Float32"]
    bf = [s.v for s in decl if s.dtype == "BFloat16"]
    assert [lay[v] for v in f32[:8]] == ["align"] * 8          # sum, sumSq, tmpSum, tmpSqSum, mean, meanSq, var, invStd
    assert [lay[v] for v in f32[8:]] == ["ortho"] * 2          # weightF, biasF
    assert [lay[v] for v in bf] == ["ortho"] * 2               # weightRV, biasRV
    src = dsl.emit_kernel(k)
    assert "rv<bf16, 64, vlayout::ortho>" in src and "rv<float, 64, vlayout::align>" in src
    assert "wave::row_broadcast<op_mul>(" in src and "wave::row_broadcast<op_add>(" in src


def test_conflicting_vector_use_is_an_error():
    k = dsl.KernelBuilder("conflict")
    t = k.allocRT("Float32", 64, 64)
    v = k.allocRV("Float32", 64)
    k.rowSum(v, t)          # align
    k.mulRow(t, t, v)       # ortho
    with pytest.raises(dsl.LayoutConflict, match="RV layout conflict for v1"):
        dsl.emit_kernel(k.build())


def test_nvidia_only_statements_are_refused_and_mma_bookkeeping_is_a_no_op():
    k = dsl.KernelBuilder("tma")
    a = k.allocST("BFloat16", 64, 64)
    k.emit(stmt("tmaExpect", a.id, 4096))
    with pytest.raises(dsl.UnsupportedStatement, match="tmaExpect"):
        dsl.emit_kernel(k.build())
    k = dsl.KernelBuilder("fence")
    k.emit(stmt("mmaCommitGroup"))
    k.emit(stmt("mmaAsyncWait", 0))
    assert dsl.emit_kernel(k.build()).count("nothing to do") == 2
    # the TMA prefetch hint changes no value: it is dropped, not refused
    k = dsl.KernelBuilder("hint")
    a = k.allocST("BFloat16", 64, 64)
    k.emit(stmt("prefetch", a.id))
    assert "a hint, nothing to do" in dsl.emit_kernel(k.build())


def test_launcher_text():
    tu = dsl.emit_translation_unit([kernels.rotaryFwd()])
    assert ('extern "C" int tyr_launch_rotaryFwd(void* x_ptr, const int64_t* x_ptr_shape, int x_ptr_ndim, '
            "void* sin_ptr") in tu
    assert "uint64_t _seq_len, uint64_t _head_dim, uint64_t grid_x" in tu
    assert "dim3(64 * waves)" in tu
    # the Lean-facing wrapper keeps the reference's signature and messages (Attribute.lean:334-336, 344-352)
    assert 'extern "C" lean_object* lean_launch_rotaryFwd(b_lean_obj_arg x_ptr, b_lean_obj_arg sin_ptr' in tu
    for msg in ["x_ptr must be a CUDA tensor", "x_ptr must be contiguous", "x_ptr must have dim <= 4"]:
        assert msg in tu


def test_emitted_kernels_compile_for_gfx950(tmp_path):
    src = dsl_build.emit_sources(str(tmp_path / "k.hip"))
    cmd = [dsl_build.HIPCC] + dsl_build.HIPFLAGS + ["-I", dsl_build.CSRC, "-c", "--cuda-device-only", src, "-o",
                                                    str(tmp_path / "k.o")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    assert os.path.getsize(tmp_path / "k.o") > 0


def test_committed_header_matches_the_emitter_and_the_library_exports_it():
    import ctypes
    from tyr_amd.dsl import runtime
    text = open(dsl_build.HEADER_PATH).read()
    assert text == dsl_build.header_text(), "regenerate include/tyr_dsl_kernels.h: python -m tyr_amd.dsl.build"
    names = re.findall(r"\bint (tyr_launch_\w+)\(", text)
    assert names == [f"tyr_launch_{f().name}" for f in kernels.ALL]
    L = runtime.load()
    for n in names:
        assert hasattr(L, n), n


def test_launcher_validates_on_the_host():
    # no GPU needed: every call fails validation before the launch
    import ctypes
    from tyr_amd.dsl import runtime
    L = runtime.load()
    fn = L.tyr_launch_copy64x64
    i64p, vp, u64 = ctypes.POINTER(ctypes.c_int64), ctypes.c_void_p, ctypes.c_uint64
    fn.argtypes = [vp, i64p, ctypes.c_int, vp, i64p, ctypes.c_int] + [u64] * 7 + [vp]
    fn.restype = ctypes.c_int
    shape = (ctypes.c_int64 * 4)(1, 1, 64, 64)
    p = vp(0x1000)
    assert fn(None, shape, 4, p, shape, 4, 1, 1, 1, 128, 1, 1, 0, None) == -2          # null tensor
    assert fn(p, shape, 5, p, shape, 4, 1, 1, 1, 128, 1, 1, 0, None) == -2             # rank > 4
    assert fn(p, shape, 4, p, shape, 4, 0, 1, 1, 128, 1, 1, 0, None) == -2             # empty grid
    assert fn(p, shape, 4, p, shape, 4, 1, 1, 1, 0, 1, 1, 0, None) == -2               # empty block
    assert fn(p, shape, 4, p, shape, 4, 1, 1, 1, 256, 1, 1, 0, None) == -2             # more warps than compiled for


def test_statement_coverage_programs_lower_and_are_built():
    # every statement kind the emitter lowers appears in some program that runs on the GPU tests
    from tests import dsl_op_programs as op_programs
    from tyr_amd.dsl import runtime
    from tyr_amd.dsl.emit import NO_OPS, NVIDIA_ONLY
    used = set()
    for f in kernels.ALL + op_programs.ALL:
        k = f()
        dsl.emit_kernel(k)
        used |= {s.op for s in walk(k.body)}
    lowered = set(KSTMT_FIELDS) - NVIDIA_ONLY - NO_OPS
    assert lowered - used == set(), lowered - used
    L = op_programs.load()
    for f in op_programs.ALL:
        assert hasattr(L, f"tyr_launch_{f().name}")


def test_write_after_read_hazards_on_shared_tiles_get_barriers():
    # LayerNorm reuses one LDS tile for x, residual and the output without barriers between a read
    # and the next overwrite (the reference launches it with one warp for that reason); the emitter
    # closes exactly those gaps, also across the loop back-edge, and adds nothing where the program
    # already synchronises
    src = dsl.emit_kernel(kernels.tkFusedLayerNormResidual1024())
    assert src.count("// inserted:") == 5
    loop = src[src.index("Pass 1"):src.index("Pass 2")]
    first = loop[loop.index("{"):]
    assert first.lstrip("{\n ").startswith("wave::sync();  // inserted")      # back-edge: tile read at the end of the previous pass
    assert dsl.emit_kernel(kernels.tkFlashAttnFwd2BlockLse(), share_lds=False).count("// inserted:") == 0
    assert dsl.emit_kernel(kernels.tkFusedLayerNormResidual1024(), hazard_barriers=False).count("// inserted:") == 0
    # a conditional cannot hold a barrier: it goes in front of the conditional
    k = dsl.KernelBuilder("cond")
    g = k.gptr("Float32", "g")
    c = k.blockCoord2D()
    t = k.allocRT("Float32", 64, 64)
    s_ = k.allocST("Float32", 64, 64)
    k.loadGlobal(s_, g, c)
    k.load(t, s_)
    with k.ifThen(k.scalarCompare("Eq", c.r, c.c)):
        k.store(s_, t)
    text = dsl.emit_kernel(k.build())
    assert text.index("// inserted:") < text.index("if (")


def test_global_tiles_of_a_loop_are_requested_one_iteration_ahead():
    # simpleGemm (Examples.lean:23-65) loads its A and B tiles at the top of the k loop: the emitter
    # splits each load into the global read (into registers, issued for iteration i+1 after the first
    # barrier of iteration i) and the write to LDS at the position of the original statement
    src = dsl.emit_kernel(kernels.simpleGemm())
    assert src.count("wave::gfrag<bf16, 64, 64>") == 2
    assert src.count("wave::gload(") == 4 and src.count("wave::sstore(") == 2
    loop = src[src.index("for (int"):]
    assert loop.index("wave::sstore(") < loop.index("wave::sync();") < loop.index("wave::gload(") < loop.index("wave::mma_AB(")
    plain = dsl.emit_kernel(kernels.simpleGemm(), prefetch_global_loads=False)
    assert "gload" not in plain and plain.count("wave::load(") == 4
    # a loop that also writes global memory keeps its loads where the program has them
    k = dsl.KernelBuilder("copy_rows")
    g, h = k.gptr("BFloat16", "src"), k.gptr("BFloat16", "dst")
    c = k.blockCoord2D()
    s_ = k.allocST("BFloat16", 64, 64)
    with k.krange(0, 4) as i:
        at = type(c)(c.b, c.d, i.id, c.c)
        k.loadGlobal(s_, g, at)
        k.sync()
        k.storeGlobal(h, s_, at)
        k.sync()
    assert "gload" not in dsl.emit_kernel(k.build())


def test_lds_tiles_with_disjoint_live_ranges_share_storage():
    # simpleGemm: the f32 staging tile of the result is only used after the k loop, its A and B tiles
    # only inside it -- one pool of 19,456 bytes instead of 36,864, i.e. twice the workgroups per CU
    src = dsl.emit_kernel(kernels.simpleGemm())
    assert "unsigned char tyr_lds_pool[19456];" in src
    assert src.count("tyr_lds_pool + 0)") == 2 and "tyr_lds_pool + 10240)" in src
    plain = dsl.emit_kernel(kernels.simpleGemm(), share_lds=False)
    assert "tyr_lds_pool" not in plain and plain.count("__shared__ st<") == 3
    # tiles that are live together never overlap: every pair of tiles used in one loop is disjoint
    from tyr_amd.dsl.emit import lds_plan, st_bytes
    for make in kernels.ALL:
        k = make()
        name = k.name
        plan = lds_plan(k)
        decl = {t.v: t for t in walk(k.body) if t.op == "declST"}
        for body in [t.body for t in walk(k.body) if t.op in ("forLoop", "forLoopVal")]:
            used = {a for t in walk(body) for a in t.args if isinstance(a, VarId) and a in plan}
            spans = sorted((plan[v], plan[v] + st_bytes(decl[v])) for v in used)
            assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), (name, spans)
    # a kernel whose tiles are all live together keeps its plain declarations
    assert "tyr_lds_pool" not in dsl.emit_kernel(kernels.tkFusedLayerNormResidual1024())
    # The attention forwards read their Q tile once, before the key loop, and write their O tile after it: both lie over the
    # K tile.  That costs one barrier in front of the loop (every wave has Q in registers before K(0) is written) and none
    # inside it; a plan that would put a barrier into a loop is dropped instead.
    att = dsl.emit_kernel(kernels.tkFlashAttnFwd2BlockLse())
    assert "unsigned char tyr_lds_pool[19456];" in att and att.count("// inserted:") == 1
    assert att.index("// inserted:") < att.index("for (int")
    lcf = dsl.emit_kernel(kernels.tkMhaH100LCFFwd128())
    assert "unsigned char tyr_lds_pool[71680];" in lcf               # 108,544 bytes as separate tiles: two workgroups per CU now
    # tiles read with the transposing LDS read (column-major operands of 2-byte elements) get 32 bytes of row padding, the others 16
    assert "st<bf16, 128, 128, 32>& v" in lcf and "st<bf16, 128, 128>& v" in lcf
    assert lcf.index("// inserted: a shared tile is overwritten") < lcf.index("for (int")


def test_programs_too_large_for_one_wave_are_run_by_a_wave_group():
    """The H100 bf16 GEMM surface (Bf16Gemm.lean:64-73: a 128x256 f32 accumulator) and the load-compute-finish
    attention surfaces (MhaH100LCF.lean:84-132: 128x128 / 192x64 K and V tiles beside a 64 x D accumulator) do not fit
    one wave's registers.  The emitter keeps their B operands in LDS and cuts the row-tied tiles into per-wave row
    slices; programs that fit one wave are emitted as before."""
    from tyr_amd.dsl.emit import _Emitter, peak_tile_registers, wave_group_plan, infer_rv_layouts, REG_BUDGET
    for f in kernels.ALL:
        k = f()
        w, split, streamed = wave_group_plan(k, infer_rv_layouts(k))
        groups = {"tkH100Bf16GemmFwd": (4, 1), "tkMhaH100LCFFwd64": (2, 2), "tkMhaH100LCFFwd128": (2, 2),
                  # the E4M3 GEMM surfaces: a 64 x 256 (128 x 256) f32 accumulator beside a 256 x 128 E4M3 B tile
                  "gemmFp8E4M3Fwd": (2, 1), "tkH100Fp8ScaledGemmFwd": (2, 1), "tkH100Fp8E4M3GemmFwd": (2, 1),
                  "tkB200Fp8E4M3Gemm1CtaFwd": (4, 1)}
        if k.name in groups:
            assert peak_tile_registers(k) > 512                      # more than a lane's whole register file
            assert w == groups[k.name][0]
            assert peak_tile_registers(k, split, w, set(streamed)) <= REG_BUDGET
            assert len(streamed) == groups[k.name][1]
        else:
            assert (w, split, streamed) == (1, set(), {}), k.name
    g = kernels.tkH100Bf16GemmFwd()
    text = dsl.emit_kernel(g)
    # two such workgroups fit a CU (LDS, and 256 registers per lane at two waves per SIMD): the compiler is told so
    assert "__launch_bounds__(256, 2)" in text and "const int tyr_wave = wave::index();" in text
    assert "rt<float, 32, 256, layout::row>" in text and "rt<float, 128, 256" not in text
    # global <-> LDS moves are shared out among the waves, the loop's tiles one iteration ahead
    assert "wave::gload_part(" in text and "wave::sstore_part(" in text and "wave::store_part(" in text
    assert ", tyr_wave * 32);" in text
    plain = dsl.emit_kernel(g, prefetch_global_loads=False)
    assert "wave::load_part(" in plain and "gload_part" not in plain
    assert re.search(r"wave::mma_ABt\(v\d+, v\d+, v14, v\d+\);", text)           # B operand = the LDS tile itself
    # a row slice stored to LDS is followed by a barrier before the group reads the whole tile
    i = text.index("wave::store(v17")
    assert text[i:].split("\n")[1].strip().startswith("wave::sync();")
    # the launcher starts exactly the group's wave count, whatever block shape the caller passes
    assert "const unsigned waves = 4;" in _Emitter(g).launcher_text()
    a = dsl.emit_kernel(kernels.tkMhaH100LCFFwd128())
    assert "rt<float, 32, 128, layout::row>" in a and a.count("stays in LDS") == 2
    # its K and V tiles are requested one iteration ahead although the loop body starts with register declarations
    assert a.count("wave::gload_part(") == 4 and a.count("wave::sstore_part(") == 2 and "__launch_bounds__(128, 2)" in a
    assert re.search(r"rv<float, 32, vlayout::align>", a)                         # per-row softmax state is sliced too


def test_operands_that_cannot_stay_in_lds_keep_their_registers():
    from tyr_amd.dsl.emit import streamed_operands
    # the backward program uses K both as a product's A operand and in a layout swap: it must stay a register tile
    assert streamed_operands(kernels.tkMhaH100Bwd2BlockPartials()) == {}
    # a tile whose LDS source is overwritten between its load and its product must not be streamed
    k = dsl.KernelBuilder("overwritten")
    p = k.gptr("BFloat16", "p")
    coord = k.blockCoord2D()
    a, b = k.allocRT("BFloat16", 64, 64), k.allocRT("BFloat16", 64, 64)
    acc = k.zeroRT("Float32", 64, 64)
    sa, sb = k.allocST("BFloat16", 64, 64), k.allocST("BFloat16", 64, 64)
    k.loadGlobal(sa, p, coord)
    k.loadGlobal(sb, p, coord)
    k.sync()
    k.load(a, sa)
    k.load(b, sb)
    k.loadGlobal(sb, p, coord.withRow(coord.c))      # sb changes before b is multiplied
    k.mmaT(acc, a, b, acc)
    assert streamed_operands(k.build()) == {}
