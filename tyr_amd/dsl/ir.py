"""Kernel IR of the tile DSL: the statement set of Tyr/GPU/Codegen/IR.lean:50-189 and the operation
tags of Tyr/GPU/Codegen/AST.lean, as plain Python values.

A statement is `Stmt(op, args)`: `op` is the constructor name of the reference's `KStmt`, `args` its
fields in declaration order (VarId, ints, floats, tags as strings, nested statement lists for the
control-flow constructors).  `KSTMT_FIELDS` is the constructor table; building a statement checks
the name and the field count against it, so a program that type-checks here maps one to one onto a
`KStmt` array.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, List, Tuple

# Tyr/GPU/Types.lean:21-59 -- name -> (C++ element type in emitted code, bytes)
GPU_FLOAT = {
    "Float32": ("float", 4),
    "Float16": ("half", 2),
    "BFloat16": ("bf16", 2),
    "FP8E4M3": ("fp8e4m3", 1),
    "FP8E5M2": ("fp8e5m2", 1),
    "FP8E8M0": ("fp8e8m0", 1),
    "FP4E2M1X2": ("fp4e2m1_2", 1),
}
TILE_LAYOUTS = ("Row", "Col")                                   # Types.lean:70-88
MMA_TRANSPOSE = ("AB", "ABt", "AtB", "AtBt")                     # AST.lean MMATranspose
REDUCE_OPS = ("Max", "Min", "Sum", "Prod")
REDUCE_AXES = ("Row", "Col", "Full")
BROADCAST_AXES = ("Row", "Col")
UNARY_OPS = ("Exp", "Exp2", "Log", "Log2", "Abs", "Relu", "Copy", "Neg", "Sqrt", "Rsqrt", "Tanh", "FastTanh",
             "Sigmoid", "Gelu", "Silu", "Swish", "Sin", "Cos", "Recip", "Square", "Zero", "One", "PosInfty",
             "NegInfty")
BINARY_OPS = ("Add", "Sub", "Mul", "Div", "Max", "Min")
TERNARY_OPS = ("FMA", "FMAAxBtC", "FMAAxCtB")
SCALAR_UNARY_OPS = ("Neg", "Exp")
SCALAR_COMPARE_OPS = ("Eq", "Lt", "Le", "Gt", "Ge")
SCALAR_BINARY_OPS = ("Add", "Sub", "Mul", "Div", "Mod", "Min", "Max")
LAYOUT_DIM_AXES = ("Batch", "Depth", "Rows", "Cols")
# mask tags carry their integer fields: ("Tril", d), ("RightFill", c), ("UpperRightFill", r, c), ("MakeCausal",)
MASK_OPS = ("Tril", "Triu", "MakeCausal", "MakeCausalT", "RightFill", "LeftFill", "UpperFill", "LowerFill",
            "UpperRightFill")
# IR.lean:28-48 -- scalar parameter kind -> C type of the extern / kernel signature
K_SCALAR_TYPES = {"UInt8": "uint8_t", "UInt16": "uint16_t", "UInt32": "uint32_t", "UInt64": "uint64_t",
                  "USize": "size_t", "Float": "double", "Float32": "float", "Bool": "uint8_t"}


@dataclass(frozen=True)
class VarId:
    """Tyr/GPU/Codegen/Var.lean: a numbered variable; printed as v<idx>."""
    idx: int

    @property
    def ident(self) -> str:
        return f"v{self.idx}"


# constructor -> field names, in the order of IR.lean
KSTMT_FIELDS = {
    "declRT": ("v", "dtype", "rows", "cols", "layout"),
    "declST": ("v", "dtype", "rows", "cols", "layout"),
    "declRV": ("v", "dtype", "len"),
    "declSV": ("v", "dtype", "len"),
    "declSemaphore": ("v",),
    "declGPtr": ("v", "dtype", "name"),
    "declKVal": ("v", "dtype", "name"),
    "load": ("dst", "src"),
    "store": ("dst", "src"),
    "loadAsync": ("dst", "src"),
    "storeAsync": ("dst", "src"),
    "storeAdd": ("dst", "src"),
    "storeAddAsync": ("dst", "src"),
    "storeMinAsync": ("dst", "src"),
    "prefetch": ("src",),
    "tmaExpect": ("barrier", "bytes"),
    "tmaLoad": ("dst", "src", "coord"),
    "tmaStore": ("dst", "src", "coord"),
    "loadGlobal": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "storeGlobal": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "loadGlobalAsync": ("dst", "src", "coordB", "coordD", "coordR", "coordC", "sem"),
    "storeGlobalAsync": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "storeGlobalAdd": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "layoutDim": ("dst", "src", "axis"),
    "loadVecGlobal": ("dst", "src", "offset"),
    "storeVecGlobal": ("dst", "src", "offset"),
    "storeVecGlobalAdd": ("dst", "src", "offset"),
    "loadVecGlobalCoord": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "storeVecGlobalCoord": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "storeVecGlobalAddCoord": ("dst", "src", "coordB", "coordD", "coordR", "coordC"),
    "loadScalarGlobal": ("dst", "src", "offset"),
    "storeScalarGlobal": ("dst", "src", "offset"),
    "multimemLoadReduce": ("op", "dst", "src"),
    "multimemStore": ("dst", "src"),
    "multimemRed": ("op", "dst", "src"),
    "mma": ("trans", "dst", "a", "b", "c"),
    "mm": ("trans", "dst", "a", "b"),
    "mmaFence": ("dst",),
    "mmaCommitGroup": (),
    "mmaAsyncWait": ("n",),
    "tcgen05Mma": ("trans", "dst", "a", "b", "c"),
    "cpAsyncLoad": ("dst", "src", "coordB", "coordD", "coordR", "coordC", "sem"),
    "tmaLoadAsync": ("dst", "src", "coordB", "coordD", "coordR", "coordC", "sem"),
    "unary": ("op", "dst", "src"),
    "binary": ("op", "dst", "a", "b"),
    "ternary": ("op", "dst", "a", "b", "c"),
    "scalarMul": ("dst", "src", "scalar"),
    "scalarAdd": ("dst", "src", "scalar"),
    "broadcast": ("axis", "dst", "vec"),
    "binaryBroadcast": ("op", "axis", "dst", "tile", "vec"),
    "reduce": ("op", "axis", "dst", "src"),
    "reduceAccum": ("op", "axis", "dst", "src", "accum"),
    "cumsum": ("axis", "dst", "src"),
    "cumprod": ("axis", "dst", "src"),
    "outer": ("dst", "a", "b"),
    "swapLayout": ("dst", "src"),
    "transpose": ("dst", "src"),
    "convert": ("dst", "src"),
    "mask": ("op", "dst", "src", "fillVal"),
    "sliceRows": ("dst", "src", "startRow", "numRows"),
    "sliceCols": ("dst", "src", "startCol", "numCols"),
    "concatCols": ("dst", "left", "right"),
    "sync": ("barrierId",),
    "arrive": ("barrierId",),
    "arriveAndWait": ("barrierId",),
    "namedBarrierSync": ("id", "numThreads"),
    "namedBarrierArrive": ("id", "numThreads"),
    "warpGroupIdx": ("dst",),
    "electOneSync": ("dst",),
    "fenceViewAsyncShared": (),
    "fenceProxyAsync": (),
    "semaphore": ("op", "sem"),
    "forLoop": ("v", "lo", "hi", "body"),
    "forLoopVal": ("v", "lo", "hi", "body"),
    "ifStmt": ("cond", "thenBody", "elseBody"),
    "ifWarpGroup": ("wgIdx", "body"),
    "comment": ("text",),
    "getBlockIdx": ("dst", "axis"),
    "getThreadIdx": ("dst", "axis"),
    "constInt": ("dst", "value"),
    "constFloat": ("dst", "value"),
    "scalarUnary": ("op", "dst", "src"),
    "scalarCompare": ("op", "dst", "a", "b"),
    "scalarBinary": ("op", "dst", "a", "b"),
    "scalarSelect": ("dst", "cond", "ifTrue", "ifFalse"),
    "vecIota": ("dst", "start", "step"),
    "vecFillScalar": ("dst", "scalar"),
    "raw": ("code",),
}


@dataclass(frozen=True)
class Stmt:
    op: str
    args: Tuple[Any, ...]

    def __post_init__(self):
        fields = KSTMT_FIELDS.get(self.op)
        if fields is None:
            raise ValueError(f"unknown statement constructor {self.op!r}")
        if len(fields) != len(self.args):
            raise ValueError(f"{self.op} takes {len(fields)} fields {fields}, got {len(self.args)}")

    def __getattr__(self, name):
        fields = KSTMT_FIELDS[object.__getattribute__(self, "op")]
        if name in fields:
            return object.__getattribute__(self, "args")[fields.index(name)]
        raise AttributeError(name)


def stmt(op: str, *args) -> Stmt:
    return Stmt(op, tuple(tuple(a) if isinstance(a, list) else a for a in args))


@dataclass(frozen=True)
class KParam:
    """IR.lean:191-197."""
    name: str
    dtype: str
    isPointer: bool = False
    scalarTy: str = "UInt64"


@dataclass
class Kernel:
    """IR.lean:199-206; `arch` is "GFX950" for everything emitted here."""
    name: str
    arch: str
    params: List[KParam]
    body: List[Stmt] = field(default_factory=list)
    sharedMemBytes: int = 0


def walk(body):
    """Every statement of a body, nested bodies included, in program order."""
    for s in body:
        yield s
        for a in s.args:
            if isinstance(a, tuple) and a and isinstance(a[0], Stmt):
                yield from walk(a)
