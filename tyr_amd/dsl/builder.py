"""Kernel builder: the Python counterpart of the reference's `KernelM` monad and its operation
vocabulary (Tyr/GPU/Codegen/Monad.lean, Ops.lean, GlobalLayout.lean, Loop.lean, Macros.lean).

Method names, argument order and the statements they append are those of the reference functions
they cite, so a kernel written against this class reads like its Lean original and lowers to the
same `KStmt` sequence.
"""
from __future__ import annotations

import contextlib
from dataclasses import dataclass, replace
from typing import List, Optional

from .ir import GPU_FLOAT, K_SCALAR_TYPES, TILE_LAYOUTS, KParam, Kernel, Stmt, VarId, stmt


@dataclass(frozen=True)
class RT:          # Tyr/GPU/Codegen/TileTypes.lean: register tile
    id: VarId
    dtype: str
    rows: int
    cols: int
    layout: str = "Row"


@dataclass(frozen=True)
class ST:          # shared (LDS) tile
    id: VarId
    dtype: str
    rows: int
    cols: int
    layout: str = "Row"


@dataclass(frozen=True)
class RV:
    id: VarId
    dtype: str
    len: int


@dataclass(frozen=True)
class SV:
    id: VarId
    dtype: str
    len: int


@dataclass(frozen=True)
class GPtr:
    id: VarId
    dtype: str
    name: str


@dataclass(frozen=True)
class KVal:
    id: VarId
    scalarTy: str
    name: str


@dataclass(frozen=True)
class KIdx:        # Loop.lean:36-42
    id: VarId


@dataclass(frozen=True)
class RTileCoord:  # GlobalLayout.lean:63-70, 408-414
    b: VarId
    d: VarId
    r: VarId
    c: VarId

    def withRow(self, new_r: VarId) -> "RTileCoord":
        return replace(self, r=new_r)

    def withCol(self, new_c: VarId) -> "RTileCoord":
        return replace(self, c=new_c)


@dataclass(frozen=True)
class SoftmaxState:  # Macros.lean:86-99
    rowMax: RV
    rowSum: RV
    prevMax: RV
    scale: RV


def _vid(x) -> VarId:
    """VarId of a typed handle (KVal, KIdx, ...) or the VarId itself."""
    return x if isinstance(x, VarId) else x.id


class KernelBuilder:
    def __init__(self, name: str, arch: str = "GFX950"):
        self.name, self.arch = name, arch
        self._next = 0
        self.params: List[KParam] = []
        self._stack: List[List[Stmt]] = [[]]

    # ---- Monad.lean: freshVar / emit / buildKernelM
    def freshVar(self) -> VarId:
        v = VarId(self._next)
        self._next += 1
        return v

    def emit(self, s: Stmt) -> None:
        self._stack[-1].append(s)

    def build(self) -> Kernel:
        assert len(self._stack) == 1, "a loop body is still open"
        return Kernel(self.name, self.arch, list(self.params), list(self._stack[0]))

    # ---- parameters (Attribute.lean: GPtr / KVal binders become KParam + declGPtr / declKVal)
    def gptr(self, dtype: str, name: str) -> GPtr:
        assert dtype in GPU_FLOAT
        v = self.freshVar()
        self.params.append(KParam(name, dtype, True))
        self.emit(stmt("declGPtr", v, dtype, name))
        return GPtr(v, dtype, name)

    def kval(self, scalarTy: str, name: str) -> KVal:
        assert scalarTy in K_SCALAR_TYPES
        v = self.freshVar()
        self.params.append(KParam(name, "Float32", False, scalarTy))
        self.emit(stmt("declKVal", v, "Float32", name))
        return KVal(v, scalarTy, name)

    # ---- Ops.lean:40-101 allocation
    def allocRT(self, dtype, rows, cols, layout="Row") -> RT:
        assert dtype in GPU_FLOAT and layout in TILE_LAYOUTS
        v = self.freshVar()
        self.emit(stmt("declRT", v, dtype, rows, cols, layout))
        return RT(v, dtype, rows, cols, layout)

    def allocST(self, dtype, rows, cols, layout="Row") -> ST:
        assert dtype in GPU_FLOAT and layout in TILE_LAYOUTS
        v = self.freshVar()
        self.emit(stmt("declST", v, dtype, rows, cols, layout))
        return ST(v, dtype, rows, cols, layout)

    def allocRV(self, dtype, length) -> RV:
        v = self.freshVar()
        self.emit(stmt("declRV", v, dtype, length))
        return RV(v, dtype, length)

    def allocSV(self, dtype, length) -> SV:
        v = self.freshVar()
        self.emit(stmt("declSV", v, dtype, length))
        return SV(v, dtype, length)

    def zeroRT(self, dtype, rows, cols, layout="Row") -> RT:
        t = self.allocRT(dtype, rows, cols, layout)
        self.emit(stmt("unary", "Zero", t.id, t.id))
        return t

    def onesRT(self, dtype, rows, cols, layout="Row") -> RT:
        t = self.allocRT(dtype, rows, cols, layout)
        self.emit(stmt("unary", "One", t.id, t.id))
        return t

    def zeroRV(self, dtype, length) -> RV:
        v = self.allocRV(dtype, length)
        self.emit(stmt("unary", "Zero", v.id, v.id))
        return v

    def negInftyRV(self, dtype, length) -> RV:
        v = self.allocRV(dtype, length)
        self.emit(stmt("unary", "NegInfty", v.id, v.id))
        return v

    # ---- Ops.lean:103-128 shared <-> register
    def load(self, dst: RT, src: ST):
        self.emit(stmt("load", dst.id, src.id))

    def store(self, dst: ST, src: RT):
        self.emit(stmt("store", dst.id, src.id))

    def loadVec(self, dst: RV, src: SV):
        self.emit(stmt("load", dst.id, src.id))

    def storeVec(self, dst: SV, src: RV):
        self.emit(stmt("store", dst.id, src.id))

    # ---- GlobalLayout.lean:174-232 coordinates
    def getBlockIdxX(self) -> VarId:
        v = self.freshVar(); self.emit(stmt("getBlockIdx", v, 0)); return v

    def getBlockIdxY(self) -> VarId:
        v = self.freshVar(); self.emit(stmt("getBlockIdx", v, 1)); return v

    def getBlockIdxZ(self) -> VarId:
        v = self.freshVar(); self.emit(stmt("getBlockIdx", v, 2)); return v

    def getThreadIdxX(self) -> VarId:
        v = self.freshVar(); self.emit(stmt("getThreadIdx", v, 0)); return v

    def constIntVal(self, value: int) -> VarId:
        v = self.freshVar(); self.emit(stmt("constInt", v, int(value))); return v

    def blockCoord2D(self) -> RTileCoord:
        b = self.constIntVal(0)
        d = self.constIntVal(0)
        r = self.getBlockIdxY()
        c = self.getBlockIdxX()
        return RTileCoord(b, d, r, c)

    def rowCoord(self, r: VarId) -> RTileCoord:
        z = self.constIntVal(0)
        return RTileCoord(z, z, r, z)

    # ---- GlobalLayout.lean:277-400 global memory
    def loadGlobal(self, dst: ST, src: GPtr, coord: RTileCoord):
        self.emit(stmt("loadGlobal", dst.id, src.id, coord.b, coord.d, coord.r, coord.c))

    def storeGlobal(self, dst: GPtr, src: ST, coord: RTileCoord):
        self.emit(stmt("storeGlobal", dst.id, src.id, coord.b, coord.d, coord.r, coord.c))

    def loadVecGlobalRow(self, dst: SV, src: GPtr, coord: RTileCoord):
        self.emit(stmt("loadVecGlobal", dst.id, src.id, coord.r))

    def storeVecGlobalRow(self, dst: GPtr, src: SV, coord: RTileCoord):
        self.emit(stmt("storeVecGlobal", dst.id, src.id, coord.r))

    def loadVecGlobalCol(self, dst: SV, src: GPtr, coord: RTileCoord):
        self.emit(stmt("loadVecGlobal", dst.id, src.id, coord.c))

    def storeVecGlobalCol(self, dst: GPtr, src: SV, coord: RTileCoord):
        self.emit(stmt("storeVecGlobal", dst.id, src.id, coord.c))

    def loadVecGlobal(self, dst: SV, src: GPtr, coord: RTileCoord):
        self.emit(stmt("loadVecGlobalCoord", dst.id, src.id, coord.b, coord.d, coord.r, coord.c))

    def storeVecGlobal(self, dst: GPtr, src: SV, coord: RTileCoord):
        self.emit(stmt("storeVecGlobalCoord", dst.id, src.id, coord.b, coord.d, coord.r, coord.c))

    def storeGlobalAdd(self, dst: GPtr, src: ST, coord: RTileCoord):
        self.emit(stmt("storeGlobalAdd", dst.id, src.id, coord.b, coord.d, coord.r, coord.c))

    def storeVecGlobalAddRow(self, dst: GPtr, src: SV, coord: RTileCoord):
        self.emit(stmt("storeVecGlobalAdd", dst.id, src.id, coord.r))

    def storeVecGlobalAddCol(self, dst: GPtr, src: SV, coord: RTileCoord):
        self.emit(stmt("storeVecGlobalAdd", dst.id, src.id, coord.c))

    def storeVecGlobalAdd(self, dst: GPtr, src: SV, coord: RTileCoord):
        self.emit(stmt("storeVecGlobalAddCoord", dst.id, src.id, coord.b, coord.d, coord.r, coord.c))

    # ---- Ops.lean:684-700, 819-835 scans
    def cumsumRow(self, dst: RT, src: RT): self.emit(stmt("cumsum", "Row", dst.id, src.id))
    def cumsumCol(self, dst: RT, src: RT): self.emit(stmt("cumsum", "Col", dst.id, src.id))
    def cumprodRow(self, dst: RT, src: RT): self.emit(stmt("cumprod", "Row", dst.id, src.id))
    def cumprodCol(self, dst: RT, src: RT): self.emit(stmt("cumprod", "Col", dst.id, src.id))

    # ---- Ops.lean: products
    def mma(self, dst: RT, a: RT, b: RT, c: RT):
        self.emit(stmt("mma", "AB", dst.id, a.id, b.id, c.id))

    def mmaT(self, dst: RT, a: RT, b: RT, c: RT):
        self.emit(stmt("mma", "ABt", dst.id, a.id, b.id, c.id))

    def mmaAtB(self, dst: RT, a: RT, b: RT, c: RT):
        self.emit(stmt("mma", "AtB", dst.id, a.id, b.id, c.id))

    def mmaAtBt(self, dst: RT, a: RT, b: RT, c: RT):
        self.emit(stmt("mma", "AtBt", dst.id, a.id, b.id, c.id))

    def mm(self, dst: RT, a: RT, b: RT, trans: str = "AB"):
        self.emit(stmt("mm", trans, dst.id, a.id, b.id))

    def fma(self, dst: RT, a: RT, b: RT, c: RT):
        self.emit(stmt("ternary", "FMA", dst.id, a.id, b.id, c.id))

    # ---- Ops.lean: element-wise on tiles
    def unaryOp(self, op: str, dst, src):
        self.emit(stmt("unary", op, dst.id, src.id))

    def binaryOp(self, op: str, dst, a, b):
        self.emit(stmt("binary", op, dst.id, a.id, b.id))

    def scalarMul(self, dst, src, scalar: float):
        self.emit(stmt("scalarMul", dst.id, src.id, float(scalar)))

    def scalarAdd(self, dst, src, scalar: float):
        self.emit(stmt("scalarAdd", dst.id, src.id, float(scalar)))

    # ---- Ops.lean:559-680 reductions and broadcasts
    def _reduce(self, op, axis, dst, src):
        self.emit(stmt("reduce", op, axis, dst.id, src.id))

    def rowMax(self, dst: RV, src: RT): self._reduce("Max", "Row", dst, src)
    def rowSum(self, dst: RV, src: RT): self._reduce("Sum", "Row", dst, src)
    def rowMin(self, dst: RV, src: RT): self._reduce("Min", "Row", dst, src)
    def rowProd(self, dst: RV, src: RT): self._reduce("Prod", "Row", dst, src)
    def colMax(self, dst: RV, src: RT): self._reduce("Max", "Col", dst, src)
    def colSum(self, dst: RV, src: RT): self._reduce("Sum", "Col", dst, src)
    def colMin(self, dst: RV, src: RT): self._reduce("Min", "Col", dst, src)
    def colProd(self, dst: RV, src: RT): self._reduce("Prod", "Col", dst, src)

    def rowMaxAccum(self, dst: RV, src: RT, accum: RV):
        self.emit(stmt("reduceAccum", "Max", "Row", dst.id, src.id, accum.id))

    def rowSumAccum(self, dst: RV, src: RT, accum: RV):
        self.emit(stmt("reduceAccum", "Sum", "Row", dst.id, src.id, accum.id))

    def broadcastRow(self, dst: RT, vec: RV):
        self.emit(stmt("broadcast", "Row", dst.id, vec.id))

    def broadcastCol(self, dst: RT, vec: RV):
        self.emit(stmt("broadcast", "Col", dst.id, vec.id))

    def _bb(self, op, axis, dst, tile, vec):
        self.emit(stmt("binaryBroadcast", op, axis, dst.id, tile.id, vec.id))

    def addRow(self, dst, tile, vec): self._bb("Add", "Row", dst, tile, vec)
    def subRow(self, dst, tile, vec): self._bb("Sub", "Row", dst, tile, vec)
    def mulRow(self, dst, tile, vec): self._bb("Mul", "Row", dst, tile, vec)
    def divRow(self, dst, tile, vec): self._bb("Div", "Row", dst, tile, vec)
    def addCol(self, dst, tile, vec): self._bb("Add", "Col", dst, tile, vec)
    def subCol(self, dst, tile, vec): self._bb("Sub", "Col", dst, tile, vec)
    def mulCol(self, dst, tile, vec): self._bb("Mul", "Col", dst, tile, vec)
    def divCol(self, dst, tile, vec): self._bb("Div", "Col", dst, tile, vec)

    def outer(self, dst: RT, a: RV, b: RV):
        self.emit(stmt("outer", dst.id, a.id, b.id))

    # ---- Ops.lean: layout / type conversion, masks, slices
    def swapLayout(self, dst: RT, src: RT): self.emit(stmt("swapLayout", dst.id, src.id))
    def transpose(self, dst: RT, src: RT): self.emit(stmt("transpose", dst.id, src.id))
    def convert(self, dst: RT, src: RT): self.emit(stmt("convert", dst.id, src.id))
    def convertVec(self, dst: RV, src: RV): self.emit(stmt("convert", dst.id, src.id))

    def makeCausal(self, dst, src, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("MakeCausal",), dst.id, src.id, fillVal))

    def makeCausalT(self, dst, src, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("MakeCausalT",), dst.id, src.id, fillVal))

    def tril(self, dst, src, diagonal: int = 0, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("Tril", int(diagonal)), dst.id, src.id, fillVal))

    def triu(self, dst, src, diagonal: int = 0, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("Triu", int(diagonal)), dst.id, src.id, fillVal))

    def rightFill(self, dst, src, colIdx: int, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("RightFill", int(colIdx)), dst.id, src.id, fillVal))

    def leftFill(self, dst, src, colIdx: int, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("LeftFill", int(colIdx)), dst.id, src.id, fillVal))

    def upperFill(self, dst, src, rowIdx: int, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("UpperFill", int(rowIdx)), dst.id, src.id, fillVal))

    def lowerFill(self, dst, src, rowIdx: int, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("LowerFill", int(rowIdx)), dst.id, src.id, fillVal))

    def sliceRows(self, dst: RT, src: RT, startRow: int, numRows: Optional[int] = None):
        self.emit(stmt("sliceRows", dst.id, src.id, startRow, dst.rows if numRows is None else numRows))

    def sliceCols(self, dst: RT, src: RT, startCol: int, numCols: Optional[int] = None):
        self.emit(stmt("sliceCols", dst.id, src.id, startCol, dst.cols if numCols is None else numCols))

    def concatCols(self, dst: RT, left: RT, right: RT):
        self.emit(stmt("concatCols", dst.id, left.id, right.id))

    # ---- Ops.lean:229-303 vectors
    def copyVec(self, dst, src): self.unaryOp("Copy", dst, src)
    def zeroVec(self, dst): self.unaryOp("Zero", dst, dst)
    def addVec(self, dst, a, b): self.binaryOp("Add", dst, a, b)
    def subVec(self, dst, a, b): self.binaryOp("Sub", dst, a, b)
    def mulVec(self, dst, a, b): self.binaryOp("Mul", dst, a, b)
    def divVec(self, dst, a, b): self.binaryOp("Div", dst, a, b)
    def scalarMulVec(self, dst, src, scalar): self.scalarMul(dst, src, scalar)
    def scalarAddVec(self, dst, src, scalar): self.scalarAdd(dst, src, scalar)
    def expVec(self, dst, src): self.unaryOp("Exp", dst, src)
    def logVec(self, dst, src): self.unaryOp("Log", dst, src)
    def rsqrtVec(self, dst, src): self.unaryOp("Rsqrt", dst, src)

    # ---- synchronisation, comments, raw code
    def sync(self, barrierId: int = 0): self.emit(stmt("sync", barrierId))
    def comment(self, text: str): self.emit(stmt("comment", text))
    def emitRaw(self, code: str): self.emit(stmt("raw", code))

    # ---- Loop.lean: `for i in krange lo hi do body`
    @contextlib.contextmanager
    def krange(self, lo: int, hi: int):
        v = self.freshVar()
        self._stack.append([])
        try:
            yield KIdx(v)
        finally:
            body = self._stack.pop()
            self.emit(stmt("forLoop", v, lo, hi, body))

    # ---- Loop.lean:68, 142-145: `for i in kvrange lo n do body` with a runtime bound
    @contextlib.contextmanager
    def kvrange(self, lo: int, hi):
        v = self.freshVar()
        self._stack.append([])
        try:
            yield KIdx(v)
        finally:
            body = self._stack.pop()
            self.emit(stmt("forLoopVal", v, lo, _vid(hi), body))

    # ---- IR.lean:179 ifStmt.  `with k.ifThen(c): ...` then optionally `with k.orElse(): ...` right after it
    @contextlib.contextmanager
    def ifThen(self, cond):
        self._stack.append([])
        try:
            yield
        finally:
            body = self._stack.pop()
            self.emit(stmt("ifStmt", _vid(cond), body, []))

    @contextlib.contextmanager
    def orElse(self):
        last = self._stack[-1][-1]
        assert last.op == "ifStmt" and not last.elseBody, "orElse follows an ifThen block"
        self._stack.append([])
        try:
            yield
        finally:
            body = self._stack.pop()
            self._stack[-1][-1] = stmt("ifStmt", last.cond, list(last.thenBody), body)

    # ---- Ops.lean:132-227 runtime scalars
    def constFloatVal(self, value: float, name: str = "const_f") -> KVal:
        v = self.freshVar(); self.emit(stmt("constFloat", v, float(value))); return KVal(v, "Float32", name)

    def loadFloat32Scalar(self, src: GPtr, offset, name: str = "load_f32") -> KVal:
        v = self.freshVar(); self.emit(stmt("loadScalarGlobal", v, src.id, _vid(offset))); return KVal(v, "Float32", name)

    def storeFloat32Scalar(self, dst: GPtr, offset, src):
        self.emit(stmt("storeScalarGlobal", dst.id, _vid(src), _vid(offset)))

    def scalarUnary(self, op: str, src, name: str = "scalar_unary") -> KVal:
        v = self.freshVar(); self.emit(stmt("scalarUnary", op, v, _vid(src))); return KVal(v, "Float32", name)

    def scalarCompare(self, op: str, a, b, name: str = "scalar_cmp") -> KVal:
        v = self.freshVar(); self.emit(stmt("scalarCompare", op, v, _vid(a), _vid(b))); return KVal(v, "Bool", name)

    def scalarBinary(self, op: str, a, b, name: str = "scalar_binary") -> KVal:
        v = self.freshVar(); self.emit(stmt("scalarBinary", op, v, _vid(a), _vid(b)))
        return KVal(v, getattr(a, "scalarTy", "UInt32"), name)

    def scalarSelect(self, cond, ifTrue, ifFalse, name: str = "scalar_select") -> KVal:
        v = self.freshVar(); self.emit(stmt("scalarSelect", v, _vid(cond), _vid(ifTrue), _vid(ifFalse)))
        return KVal(v, getattr(ifTrue, "scalarTy", "UInt32"), name)

    def iotaVec(self, dst: RV, start: float = 0.0, step: float = 1.0):
        self.emit(stmt("vecIota", dst.id, float(start), float(step)))

    def fillVecScalar(self, dst: RV, scalar):
        self.emit(stmt("vecFillScalar", dst.id, _vid(scalar)))

    # ---- Ops.lean:912-938 dimensions of a global layout
    def layoutDim(self, src: GPtr, axis: str, name: str = "layout_dim") -> KVal:
        v = self.freshVar(); self.emit(stmt("layoutDim", v, src.id, axis)); return KVal(v, "UInt32", name)

    def layoutBatch(self, src): return self.layoutDim(src, "Batch", "batch")
    def layoutDepth(self, src): return self.layoutDim(src, "Depth", "depth")
    def layoutRows(self, src): return self.layoutDim(src, "Rows", "rows")
    def layoutCols(self, src): return self.layoutDim(src, "Cols", "cols")

    def upperRightFill(self, dst, src, row: int, col: int, fillVal: Optional[float] = None):
        self.emit(stmt("mask", ("UpperRightFill", int(row), int(col)), dst.id, src.id, fillVal))

    # ---- Macros.lean:101-163 online softmax
    def allocSoftmaxState(self, dtype, rows) -> SoftmaxState:
        rowMax = self.negInftyRV(dtype, rows)
        rowSum = self.zeroRV(dtype, rows)
        prevMax = self.allocRV(dtype, rows)
        scale = self.allocRV(dtype, rows)
        return SoftmaxState(rowMax, rowSum, prevMax, scale)

    def onlineSoftmax(self, scores: RT, output: RT, state: SoftmaxState):
        self.copyVec(state.prevMax, state.rowMax)
        self.rowMaxAccum(state.rowMax, scores, state.rowMax)
        self.subVec(state.scale, state.prevMax, state.rowMax)
        self.expVec(state.scale, state.scale)
        self.mulCol(output, output, state.scale)
        self.mulVec(state.rowSum, state.rowSum, state.scale)
        self.subCol(scores, scores, state.rowMax)
        self.exp(scores, scores)
        self.rowSumAccum(state.rowSum, scores, state.rowSum)

    def finalizeSoftmax(self, output: RT, state: SoftmaxState):
        self.divCol(output, output, state.rowSum)

    def computeLSE(self, state: SoftmaxState) -> RV:
        lse = self.allocRV(state.rowSum.dtype, state.rowSum.len)
        self.logVec(lse, state.rowSum)
        self.addVec(lse, lse, state.rowMax)
        return lse


def _add_elementwise_names():
    # Ops.lean:430-540: one method per unary / binary tag
    unary = {"exp": "Exp", "exp2": "Exp2", "log": "Log", "sqrt": "Sqrt", "rsqrt": "Rsqrt", "tanh": "Tanh",
             "fastTanh": "FastTanh", "sigmoid": "Sigmoid", "gelu": "Gelu", "relu": "Relu", "neg": "Neg",
             "abs": "Abs", "copy": "Copy", "sin": "Sin", "cos": "Cos", "silu": "Silu", "swish": "Swish",
             "recip": "Recip", "square": "Square"}
    for name, tag in unary.items():
        setattr(KernelBuilder, name, (lambda tag: lambda self, dst, src: self.unaryOp(tag, dst, src))(tag))
    setattr(KernelBuilder, "zero", lambda self, dst: self.unaryOp("Zero", dst, dst))
    setattr(KernelBuilder, "ones", lambda self, dst: self.unaryOp("One", dst, dst))
    for name, tag in {"add": "Add", "sub": "Sub", "mul": "Mul", "div": "Div", "max": "Max", "min": "Min"}.items():
        setattr(KernelBuilder, name, (lambda tag: lambda self, dst, a, b: self.binaryOp(tag, dst, a, b))(tag))


_add_elementwise_names()
