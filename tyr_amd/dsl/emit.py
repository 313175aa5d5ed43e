"""HIP emitter for the tile DSL: `Kernel` -> one gfx950 translation unit.

The counterpart of the reference's CUDA emitter (Tyr/GPU/Codegen/EmitNew.lean:207-700 prints one
ThunderKittens call per statement; Tyr/GPU/Codegen/Attribute.lean:318-386 prints the launcher).
Here a statement becomes one call into the wave-level tile vocabulary of
`tyr_amd/csrc/tile/tyr_tile.hpp`, and the launcher is a C-ABI function over raw pointers plus, for a
build that has Lean and LibTorch headers, the `lean_launch_<kernel>` wrapper with the reference's
signature and error strings.

Statements that only exist for NVIDIA hardware paths (TMA, multimem, tcgen05, semaphores, named
barriers, warp-group election) raise `UnsupportedStatement`; the asynchronous-MMA bookkeeping
statements are no-ops because an MFMA is complete when its result is read, and the prefetch hint is
a no-op because it changes no value.
"""
from __future__ import annotations

from typing import Any, Dict, List

from .ir import GPU_FLOAT, K_SCALAR_TYPES, Kernel, Stmt, VarId, walk


class UnsupportedStatement(NotImplementedError):
    pass


class LayoutConflict(ValueError):
    pass


CPP_TYPE = {"Float32": "float", "BFloat16": "bf16", "FP8E4M3": "fp8e4m3"}
UNARY = {"Exp": "op_exp", "Exp2": "op_exp2", "Log": "op_log", "Log2": "op_log2", "Abs": "op_abs", "Relu": "op_relu",
         "Copy": "op_copy", "Neg": "op_neg", "Sqrt": "op_sqrt", "Rsqrt": "op_rsqrt", "Tanh": "op_tanh",
         "FastTanh": "op_tanh", "Sigmoid": "op_sigmoid", "Gelu": "op_gelu", "Silu": "op_silu", "Swish": "op_silu",
         "Sin": "op_sin", "Cos": "op_cos", "Recip": "op_recip", "Square": "op_square", "Zero": "op_zero",
         "One": "op_one", "PosInfty": "op_pos_infty", "NegInfty": "op_neg_infty"}
BINARY = {"Add": "op_add", "Sub": "op_sub", "Mul": "op_mul", "Div": "op_div", "Max": "op_max", "Min": "op_min"}
REDUCE = {"Max": "op_max", "Min": "op_min", "Sum": "op_add", "Prod": "op_mul"}
MASK = {"MakeCausal": "keep_causal", "MakeCausalT": "keep_causal_t", "Tril": "keep_tril", "Triu": "keep_triu",
        "RightFill": "keep_right_fill", "LeftFill": "keep_left_fill", "UpperFill": "keep_upper_fill",
        "LowerFill": "keep_lower_fill"}
NO_OPS = {"mmaFence", "mmaCommitGroup", "mmaAsyncWait", "fenceViewAsyncShared", "fenceProxyAsync", "prefetch"}
NVIDIA_ONLY = {"declSemaphore", "loadAsync", "storeAsync", "storeAdd", "storeAddAsync", "storeMinAsync",
               "tmaExpect", "tmaLoad", "tmaStore", "loadGlobalAsync", "storeGlobalAsync",
               "multimemLoadReduce", "multimemStore", "multimemRed",
               "tcgen05Mma", "cpAsyncLoad", "tmaLoadAsync", "arrive", "arriveAndWait", "namedBarrierSync",
               "namedBarrierArrive", "warpGroupIdx", "electOneSync", "semaphore", "ifWarpGroup"}


def _cpp_type(dtype: str) -> str:
    if dtype not in CPP_TYPE:
        raise UnsupportedStatement(f"element type {dtype} has no gfx950 tile type yet (have {sorted(CPP_TYPE)})")
    return CPP_TYPE[dtype]


def _flt(x: float) -> str:
    if x != x:
        return "NAN"
    if x in (float("inf"), float("-inf")):
        return "INFINITY" if x > 0 else "-INFINITY"
    return repr(float(x)) + "f"


def infer_rv_layouts(kernel: Kernel) -> Dict[VarId, str]:
    """align / ortho for every register vector (the reference infers naive / ortho / align the
    same way, EmitNew.lean:100-200): what a vector is reduced from or broadcast along fixes its
    layout, and element-wise vector statements tie their operands together."""
    rvs = {s.v for s in walk(kernel.body) if s.op == "declRV"}
    parent = {v: v for v in rvs}

    def find(v):
        while parent[v] != v:
            parent[v] = parent[parent[v]]
            v = parent[v]
        return v

    want: Dict[VarId, set] = {}

    def need(v, lay):
        if v in rvs:
            want.setdefault(v, set()).add(lay)

    def tie(*vs):
        vs = [v for v in vs if v in rvs]
        for v in vs[1:]:
            parent[find(v)] = find(vs[0])

    for s in walk(kernel.body):
        if s.op in ("reduce", "reduceAccum") and s.axis == "Full":
            if s.op == "reduceAccum":                    # any layout serves: the result lands in every element
                tie(s.dst, s.accum)
        elif s.op in ("cumsum", "cumprod") and s.axis == "Full":
            need(s.dst, "align")
            need(s.src, "align")
        elif s.op == "reduce":
            need(s.dst, "align" if s.axis == "Row" else "ortho")
        elif s.op == "reduceAccum":
            lay = "align" if s.axis == "Row" else "ortho"
            need(s.dst, lay)
            need(s.accum, lay)
        elif s.op in ("broadcast", "binaryBroadcast"):
            need(s.vec, "align" if s.axis == "Col" else "ortho")
        elif s.op == "outer":
            need(s.a, "align")
            need(s.b, "ortho")
        elif s.op in ("unary", "convert", "scalarMul", "scalarAdd"):
            tie(s.dst, s.src)
        elif s.op == "binary":
            tie(s.dst, s.a, s.b)
    groups: Dict[VarId, set] = {}
    for v, lays in want.items():
        groups.setdefault(find(v), set()).update(lays)
    out = {}
    for v in rvs:
        lays = groups.get(find(v), set())
        if len(lays) > 1:
            raise LayoutConflict(f"RV layout conflict for {v.ident}")
        out[v] = next(iter(lays)) if lays else "align"
    return out


_DTYPE_BYTES = {"Float32": 4, "BFloat16": 2, "Float16": 2, "FP8E4M3": 1, "FP8E5M2": 1}

# Padding bytes behind every row of an LDS tile (a multiple of 16: rows stay 16-byte aligned for the 16-byte global <-> LDS
# moves).  The fragment accesses of this tile library are 8 bytes per lane, 16 lanes to an LDS cycle; which row pitch keeps
# those apart depends on who the 16 lanes are:
#   row fragments (lane = row; tiles declared Row): 16 consecutive rows x 2 dwords -- a pitch of 4 dwords mod 64 is conflict-free
#     on 64 banks, which is what a row of 128 / 256 / 512 bytes gets from 16 bytes of padding;
#   transposing reads (tiles declared Col, bf16): 4 consecutive rows x four 8-byte column groups -- the rows must land 8 dwords
#     apart mod 32, i.e. 32 bytes of padding behind rows of 64 / 128 / 256 bytes.
_PAD_OVERRIDE = {}


def st_pad_bytes(d: Stmt) -> int:
    """Row padding of the LDS tile declared by `d` (a declST statement)."""
    key = (d.dtype, d.layout)
    if key in _PAD_OVERRIDE:
        return _PAD_OVERRIDE[key]
    if d.layout == "Col" and _DTYPE_BYTES.get(d.dtype) == 2:
        return 32
    return 16


def st_bytes(d: Stmt) -> int:
    """Bytes an LDS tile occupies (rounded up to 16)."""
    return (d.rows * (d.cols * _DTYPE_BYTES[d.dtype] + st_pad_bytes(d)) + 15) // 16 * 16


def _st_uses(s: Stmt, tiles) -> set:
    """LDS tiles a (non-compound) statement touches."""
    out = set()
    for a in s.args:
        if isinstance(a, VarId) and a in tiles:
            out.add(a)
    return out


def lds_plan(kernel: Kernel) -> Dict[VarId, int]:
    """Byte offsets of the LDS tiles in one pool, or {} when sharing storage saves nothing.

    Tiles whose live ranges (first to last use in program order; a use inside a loop counts for the
    whole loop) do not intersect may occupy the same bytes: a GEMM's output staging tile is only
    used after the loop that uses its operand tiles.  Less LDS per workgroup is more workgroups per
    CU."""
    decl = {s.v: s for s in walk(kernel.body) if s.op == "declST"}
    if len(decl) < 2:
        return {}
    size = {}
    for v, d in decl.items():
        b = _DTYPE_BYTES.get(d.dtype)
        if b is None:
            return {}
        size[v] = st_bytes(d)
    live: Dict[VarId, List[int]] = {}
    pos = [0]

    def touch(v, a, b):
        r = live.setdefault(v, [a, b])
        r[0], r[1] = min(r[0], a), max(r[1], b)

    def run(body):
        for s in body:
            pos[0] += 1
            if s.op in ("forLoop", "forLoopVal"):
                start = pos[0]
                before = {v: list(r) for v, r in live.items()}
                run(s.body)
                end = pos[0]
                for v, r in live.items():
                    if before.get(v) != r:               # used inside the loop: live for all of it
                        touch(v, start, end)
            elif s.op == "ifStmt":
                run(s.thenBody)
                run(s.elseBody)
            elif s.op != "declST":
                for v in _st_uses(s, decl):
                    touch(v, pos[0], pos[0])

    run(kernel.body)
    placed: Dict[VarId, int] = {}
    for v in sorted(decl, key=lambda t: -size[t]):
        if v not in live:
            live[v] = [0, 0]
        off = 0
        while True:
            clash = [u for u in placed
                     if not (live[u][1] < live[v][0] or live[v][1] < live[u][0])
                     and off < placed[u] + size[u] and placed[u] < off + size[v]]
            if not clash:
                break
            off = max(placed[u] + size[u] for u in clash)
        placed[v] = off
    total = max(placed[v] + size[v] for v in placed)
    if total >= sum(size.values()):
        return {}
    return placed


def _lds_regions(kernel: Kernel, plan: Dict[VarId, int]) -> Dict[VarId, Any]:
    """Tiles that share bytes are one object for the hazard analysis."""
    if not plan:
        return {}
    decl = {s.v: s for s in walk(kernel.body) if s.op == "declST"}
    size = {v: st_bytes(d) for v, d in decl.items()}
    root = {v: v for v in plan}

    def find(v):
        while root[v] != v:
            v = root[v]
        return v
    vs = list(plan)
    for i, a in enumerate(vs):
        for b in vs[i + 1:]:
            if plan[a] < plan[b] + size[b] and plan[b] < plan[a] + size[a]:
                root[find(a)] = find(b)
    return {v: ("lds", find(v).ident) for v in vs}


def shared_hazard_barriers(kernel: Kernel, regions: Dict[VarId, Any] = None, streamed: Dict[VarId, VarId] = None) -> set:
    """ids of the statements that need a workgroup barrier in front of them.

    Every wave of a workgroup runs the whole tile program, so the LDS tiles and vectors are shared
    by waves that drift apart between barriers.  Overwriting one of them while another wave may still
    be reading its previous contents is a write-after-read hazard; the reference's programs leave
    several of those to timing (and launch a single warp where it matters,
    Examples/GPU/RunLayerNorm.lean:66-67).  Here the emitter closes them: a barrier goes in front of
    any statement that overwrites a shared object read since the last barrier, loop back-edges
    included.  (Read-after-write needs nothing: all waves write identical data and a wave reads
    after its own write.)  A conditional body cannot hold a barrier, so the barrier goes in front of
    the conditional.  Where only what was read *before* a loop is overwritten inside it, one barrier goes
    in front of the loop instead of one into every iteration."""
    shared = {s.v for s in walk(kernel.body) if s.op in ("declST", "declSV")}
    regions = regions or {}

    def obj(v):
        return {regions.get(v, v)} if v in shared else set()

    streamed = streamed or {}

    def rw(s: Stmt):
        if s.op == "load" and s.dst in streamed:
            return (set(), set())                        # not read here: the products read the LDS tile themselves
        if s.op == "mma" and s.b in streamed:
            return (obj(streamed[s.b]), set())
        if s.op == "load":
            return (obj(s.src), set())
        if s.op == "store":
            return (set(), obj(s.dst))
        if s.op in ("loadGlobal", "loadVecGlobal", "loadVecGlobalCoord"):
            return (set(), obj(s.dst))
        if s.op in ("storeGlobal", "storeVecGlobal", "storeVecGlobalCoord", "storeGlobalAdd", "storeVecGlobalAdd",
                    "storeVecGlobalAddCoord"):
            return (obj(s.src), set())
        if s.op == "swapLayout" or (s.op == "transpose"):
            return ({("scratch", id(s))}, {("scratch", id(s))})      # the statement's own staging tile
        return (set(), set())

    def all_rw(body):
        r, w = set(), set()
        for s in walk(body):
            a, b = rw(s)
            r |= a
            w |= b
        return r, w

    def run(body, pending: set, marks) -> set:
        """Walks a statement list; `marks` (a set, or None for a dry run) collects the statements that need a barrier."""
        for s in body:
            if s.op == "sync":
                pending = set()
            elif s.op in ("forLoop", "forLoopVal"):
                # hazards of the loop by itself (entry state = what its own back edge brings) ...
                own = set()
                run(s.body, run(s.body, set(), None), own)
                # ... and with what is pending from before the loop
                full = set()
                end = run(s.body, pending | run(s.body, set(pending), None), full)   # second pass sees the back-edge
                if full != own:
                    # reads from before the loop are overwritten inside it: one barrier in front of the loop
                    if marks is not None:
                        marks.add(id(s))
                        marks |= own
                    pending = run(s.body, run(s.body, set(), None), None)
                else:
                    if marks is not None:
                        marks |= full
                    pending = pending | end
            elif s.op == "ifStmt":
                r, w = all_rw(s.thenBody + s.elseBody)
                if w & pending:
                    if marks is not None:
                        marks.add(id(s))
                    pending = set()
                pending = pending | r
            else:
                r, w = rw(s)
                if w & pending:
                    if marks is not None:
                        marks.add(id(s))
                    pending = set()
                pending = pending | r
        return pending

    marks = set()
    run(kernel.body, set(), marks)
    return marks


# ---------------------------------------------------------------------------- wave groups
# A program written for one warp of the reference can declare register tiles that no single wave holds
# (the H100 GEMM surface accumulates 128x256 in f32: 512 registers per lane; the D = 128 attention surface
# keeps 128x128 K and V tiles next to a 64x128 accumulator).  Such a program is run by a group of W waves:
#   * B operands that are only loaded from an LDS tile and multiplied stay in LDS ("streamed": the
#     product reads its fragments as it goes);
#   * register tiles and per-row vectors that are tied to an accumulator through their rows are cut
#     into W row slices, one per wave; loads and stores against LDS take the wave's row offset;
#   * global <-> LDS moves are shared out among the waves.
REG_BUDGET = 400          # registers per lane a plan may need for its register tiles (of 512)


def _rt_regs(d: Stmt, rows=None) -> int:
    return (rows if rows is not None else d.rows) * d.cols // 64      # one register per element per lane


def streamed_operands(kernel: Kernel) -> Dict[VarId, VarId]:
    """register tile -> LDS tile, for tiles that are defined only by `load` from LDS and used only as the B
    operand of products in the same statement list, with no write to that LDS tile in between."""
    info = {s.v: s for s in walk(kernel.body) if s.op in ("declRT", "declST")}
    uses: Dict[VarId, List[Stmt]] = {}
    for s in walk(kernel.body):
        if s.op in ("declRT", "forLoop", "forLoopVal", "ifStmt", "comment"):
            continue
        for a in s.args:
            if isinstance(a, VarId) and a in info and info[a].op == "declRT":
                uses.setdefault(a, []).append(s)
    cand = {}
    for v, us in uses.items():
        d = info[v]
        if d.dtype not in ("BFloat16", "FP8E4M3"):
            continue
        ok = True
        for u in us:
            if u.op == "load" and u.dst == v and u.src in info and info[u.src].op == "declST":
                continue
            if u.op == "mma" and u.b == v and v not in (u.dst, u.a, u.c) and (
                    (u.trans == "ABt" and d.layout == "Row") or
                    (u.trans == "AB" and d.layout == "Col" and d.dtype == "BFloat16")):
                continue
            ok = False
        if ok and any(u.op == "load" for u in us) and any(u.op == "mma" for u in us):
            cand[v] = None

    def scan(body):
        cur: Dict[VarId, VarId] = {}                     # tile -> LDS tile it currently mirrors
        for s in body:
            if s.op in ("forLoop", "forLoopVal"):
                scan(s.body)
                cur = {}
            elif s.op == "ifStmt":
                scan(s.thenBody)
                scan(s.elseBody)
                cur = {}
            elif s.op == "load" and s.dst in cand:
                cur[s.dst] = s.src
                if cand[s.dst] not in (None, s.src):
                    cand[s.dst] = False                  # mirrors two different LDS tiles: keep it in registers
                elif cand[s.dst] is None:
                    cand[s.dst] = s.src
            elif s.op == "mma" and s.b in cand:
                if s.b not in cur:
                    cand[s.b] = False                    # multiplied in another statement list than it is loaded in
            elif s.op in ("loadGlobal", "store"):
                # LDS tile overwritten: a later product of a tile that mirrors it would see the new data,
                # so that tile loses its mirror (and a product that follows disqualifies it above)
                for v in [v for v, st_ in cur.items() if st_ == s.dst]:
                    del cur[v]
    scan(kernel.body)
    return {v: st_ for v, st_ in cand.items() if st_}


def row_split_set(kernel: Kernel, rv_layout: Dict[VarId, str], streamed: Dict[VarId, VarId]):
    """Register tiles and vectors tied to a product's accumulator through their rows, or None when a
    statement touching them has no row-sliced form."""
    info = {s.v: s for s in walk(kernel.body) if s.op in ("declRT", "declRV")}
    parent = {v: v for v in info}

    def find(v):
        while parent[v] != v:
            parent[v] = parent[parent[v]]
            v = parent[v]
        return v

    def tie(*vs):
        vs = [v for v in vs if v in info]
        for v in vs[1:]:
            parent[find(v)] = find(vs[0])

    seeds = []
    for s in walk(kernel.body):
        if s.op == "mma" and s.trans in ("AB", "ABt"):
            tie(s.dst, s.a, s.c)
            seeds.append(s.dst)
        elif s.op == "mm" and s.trans in ("AB", "ABt"):
            tie(s.dst, s.a)
            seeds.append(s.dst)
        elif s.op in ("unary", "convert", "scalarMul", "scalarAdd"):
            tie(s.dst, s.src)
        elif s.op == "binary":
            tie(s.dst, s.a, s.b)
        elif s.op == "ternary":
            tie(s.dst, s.a, s.b, s.c)
        elif s.op == "binaryBroadcast":
            tie(s.dst, s.tile, *( [s.vec] if s.axis == "Col" else [] ))
        elif s.op == "broadcast" and s.axis == "Col":
            tie(s.dst, s.vec)
        elif s.op == "reduce" and s.axis == "Row":
            tie(s.dst, s.src)
        elif s.op == "reduceAccum" and s.axis == "Row":
            tie(s.dst, s.src, s.accum)
    roots = {find(v) for v in seeds}
    split = {v for v in info if find(v) in roots}
    if not split:
        return None
    plain = {"declRT", "declRV", "load", "store", "unary", "convert", "scalarMul", "scalarAdd", "binary", "ternary",
             "vecFillScalar", "comment"}
    for s in walk(kernel.body):
        touched = [a for a in s.args if isinstance(a, VarId) and a in split]
        if not touched or s.op in plain:
            continue
        if s.op in ("mma", "mm"):
            if s.trans not in ("AB", "ABt") or s.b in split:
                return None
        elif s.op == "binaryBroadcast":
            if s.axis == "Row" and s.vec in split:
                return None
        elif s.op == "broadcast":
            if s.axis != "Col":
                return None
        elif s.op in ("reduce", "reduceAccum"):
            if s.axis != "Row":
                return None
        else:
            return None                                  # masks, transposes, slices, scans ... have no sliced form yet
    for v in split:
        d = info[v]
        if d.op == "declRV" and rv_layout.get(v) != "align":
            return None
        if d.op == "declRT" and d.layout != "Row":
            return None
    return split


def peak_tile_registers(kernel: Kernel, split=frozenset(), waves: int = 1, streamed=frozenset(), packed: bool = False) -> int:
    """Most registers per lane the register tiles live at one point need (a tile lives from its first to its
    last mention; a mention inside a loop counts for the whole loop).  One register per element, or -- `packed` --
    what the elements' bytes really take (two bf16 or four fp8 values per register)."""
    decl = {s.v: s for s in walk(kernel.body) if s.op == "declRT"}
    live: Dict[VarId, List[int]] = {}
    pos = [0]

    def run(body):
        for s in body:
            pos[0] += 1
            if s.op in ("forLoop", "forLoopVal"):
                start = pos[0]
                before = {v: list(r) for v, r in live.items()}
                run(s.body)
                for v, r in live.items():
                    if before.get(v) != r and v in before:        # defined outside, used inside: live for the loop
                        r[0], r[1] = min(r[0], start), max(r[1], pos[0])
            elif s.op == "ifStmt":
                run(s.thenBody)
                run(s.elseBody)
            elif s.op != "declRT":
                for a in s.args:
                    if isinstance(a, VarId) and a in decl and a not in streamed:
                        r = live.setdefault(a, [pos[0], pos[0]])
                        r[1] = pos[0]
    run(kernel.body)
    peak = 0
    for p_ in range(1, pos[0] + 1):
        need = sum(_rt_regs(decl[v], decl[v].rows // waves if v in split else None) *
                   (_DTYPE_BYTES.get(decl[v].dtype, 4) if packed else 4) // 4 for v, r in live.items() if r[0] <= p_ <= r[1])
        peak = max(peak, need)
    return peak


def wave_group_plan(kernel: Kernel, rv_layout: Dict[VarId, str]):
    """(waves, split set, streamed map) for a program: (1, {}, {}) when one wave holds it."""
    if peak_tile_registers(kernel) <= REG_BUDGET:
        return 1, set(), {}
    streamed = streamed_operands(kernel)
    if streamed and peak_tile_registers(kernel, streamed=set(streamed)) <= REG_BUDGET:
        return 1, set(), streamed
    split = row_split_set(kernel, rv_layout, streamed)
    if split:
        decl = {s.v: s for s in walk(kernel.body) if s.op in ("declRT", "declRV")}
        for w in (2, 4):
            sizes = [(decl[v].rows if decl[v].op == "declRT" else decl[v].len) for v in split]
            if any(n % (32 * w) for n in sizes):
                continue
            if peak_tile_registers(kernel, split, w, set(streamed)) <= REG_BUDGET:
                return w, split, streamed
    return 1, set(), {}


class _Emitter:
    def __init__(self, kernel: Kernel, max_waves: int = 4, hazard_barriers: bool = True,
                 prefetch_global_loads: bool = True, share_lds: bool = True, wave_group=None,
                 fuse_online_softmax: bool = True):
        self.k = kernel
        self.fuse_online_softmax = fuse_online_softmax
        self.info: Dict[VarId, Stmt] = {}
        for s in walk(kernel.body):
            if s.op in ("declRT", "declST", "declRV", "declSV", "declGPtr", "declKVal"):
                self.info[s.v] = s
        self.rv_layout = infer_rv_layouts(kernel)
        # one wave, or a group of waves sharing the program's tiles (see wave_group_plan)
        self.waves, self.split, self.streamed = wave_group if wave_group is not None else wave_group_plan(kernel, self.rv_layout)
        self.group = self.waves > 1
        self.dirty: set = set()          # LDS objects written in shares by the group since the last barrier
        # request the next iteration's global tiles of a loop before the work of the current one
        self.prefetch_global_loads = prefetch_global_loads
        # LDS tiles with disjoint live ranges share storage
        # (only where that puts no additional barrier into a loop)
        self.lds = lds_plan(kernel) if share_lds else {}
        if self.lds:
            in_loops = {id(t) for l in walk(kernel.body) if l.op in ("forLoop", "forLoopVal") for t in walk(l.body)}
            extra = shared_hazard_barriers(kernel, _lds_regions(kernel, self.lds), self.streamed) - \
                shared_hazard_barriers(kernel, None, self.streamed)
            if extra & in_loops:
                self.lds = {}
        self.barrier_before = shared_hazard_barriers(kernel, _lds_regions(kernel, self.lds), self.streamed) \
            if hazard_barriers else set()
        # waves per workgroup the kernel is compiled for; 4 (one per SIMD) leaves every wave the
        # full 512-register file, and covers the 128-thread blocks the reference's runners launch.
        # A wave group needs exactly its own number of waves.
        self.max_waves = self.waves if self.group else max_waves
        self.min_blocks = self._blocks_per_cu()

    def _blocks_per_cu(self) -> int:
        """Workgroups per CU the kernel is compiled for.  A wave-group program runs with exactly its own number of waves, so
        when two such workgroups fit a CU -- LDS, and 256 registers per lane at two waves per SIMD -- the compiler is told to
        keep to that budget: a second resident workgroup hides the first one's global latency and its epilogue."""
        if not self.group:
            return 1
        decl = {t.v: t for t in walk(self.k.body) if t.op == "declST"}
        size = {v: st_bytes(d) for v, d in decl.items()}
        lds = max((off + size[v] for v, off in self.lds.items()), default=0) if self.lds else sum(size.values())
        if 2 * lds > 160 * 1024:
            return 1
        if 2 * self.waves <= 4:
            return 2                                     # still one wave per SIMD: the whole register file each
        regs = peak_tile_registers(self.k, self.split, self.waves, set(self.streamed), packed=True)
        for l in (t for t in walk(self.k.body) if t.op in ("forLoop", "forLoopVal")):
            if self.prefetch_global_loads:
                regs += sum(self.info[t.dst].rows * self.info[t.dst].cols * _DTYPE_BYTES[self.info[t.dst].dtype] // (256 * self.waves)
                            for t in self.prefetchable(l))
        return 2 if regs <= 248 else 1               # the rest of the 256 goes to addresses and operand fragments

    def kind(self, v: VarId) -> str:
        s = self.info.get(v)
        return s.op[4:] if s is not None else "scalar"

    def is_vec(self, v):
        return self.kind(v) in ("RV", "SV")

    # ------------------------------------------------------------------ statements
    def stmt(self, s: Stmt, ind: str) -> str:
        op, I = s.op, (lambda v: v.ident)
        if op in NVIDIA_ONLY:
            raise UnsupportedStatement(f"{op} has no gfx950 lowering")
        if op == "prefetch":
            # a hint with no effect on values (the reference prints warp::tma::prefetch, EmitNew.lean:239); the tile is
            # fetched by the load that uses it
            return f"{ind}// prefetch of {I(s.src)}: a hint, nothing to do\n"
        if op in NO_OPS:
            return f"{ind}// {op}: nothing to do, an MFMA result is complete when it is read\n"
        if op == "declRT":
            if s.v in self.streamed:
                return f"{ind}// {I(s.v)} stays in LDS: products read their fragments from {I(self.streamed[s.v])}\n"
            rows = s.rows // self.waves if s.v in self.split else s.rows
            # (value-initialised: a program that accumulates into a tile it never wrote reads zeros, not whatever the
            #  registers held; where the tile is written first the compiler drops the zeros)
            return f"{ind}rt<{_cpp_type(s.dtype)}, {rows}, {s.cols}, layout::{s.layout.lower()}> {I(s.v)}{{}};\n"
        if op == "declST":
            pad = st_pad_bytes(s)
            ty = f"st<{_cpp_type(s.dtype)}, {s.rows}, {s.cols}" + (f", {pad}>" if pad != 16 else ">")
            if s.v in self.lds:
                return f"{ind}{ty}& {I(s.v)} = *reinterpret_cast<{ty}*>(tyr_lds_pool + {self.lds[s.v]});\n"
            return f"{ind}__shared__ {ty} {I(s.v)};\n"
        if op == "declRV":
            n = s.len // self.waves if s.v in self.split else s.len
            return f"{ind}rv<{_cpp_type(s.dtype)}, {n}, vlayout::{self.rv_layout[s.v]}> {I(s.v)}{{}};\n"
        if op == "declSV":
            return f"{ind}__shared__ sv<{_cpp_type(s.dtype)}, {s.len}> {I(s.v)};\n"
        if op == "declGPtr":
            return f"{ind}// param: {_cpp_type(s.dtype)}* {s.name} ({I(s.v)})\n"
        if op == "declKVal":
            return f"{ind}// param: {s.name} ({I(s.v)})\n"
        if op in ("load", "store"):
            reg = s.dst if op == "load" else s.src
            if reg in self.streamed:
                return f"{ind}// load of {I(reg)} elided: it stays in {I(self.streamed[reg])}\n"
            if reg in self.split:                        # this wave's row slice
                d = self.info[reg]
                n = (d.rows if d.op == "declRT" else d.len) // self.waves
                return f"{ind}wave::{op}({I(s.dst)}, {I(s.src)}, tyr_wave * {n});\n"
            return f"{ind}wave::{op}({I(s.dst)}, {I(s.src)});\n"
        if op in ("loadGlobal", "storeGlobal"):
            tile = self.info[s.dst if op == "loadGlobal" else s.src]
            at = f"coord{{(int){I(s.coordB)}, (int){I(s.coordD)}, (int){I(s.coordR)} * {tile.rows}, (int){I(s.coordC)} * {tile.cols}}}"
            if self.group:                               # the group shares the move
                return (f"{ind}wave::{'load_part' if op == 'loadGlobal' else 'store_part'}({I(s.dst)}, {I(s.src)}, {at}, "
                        f"tyr_wave, {self.waves});\n")
            return f"{ind}wave::{'load' if op == 'loadGlobal' else 'store'}({I(s.dst)}, {I(s.src)}, {at});\n"
        if op in ("loadVecGlobal", "storeVecGlobal"):
            return f"{ind}wave::{'load' if op == 'loadVecGlobal' else 'store'}({I(s.dst)}, {I(s.src)}, (int){I(s.offset)});\n"
        if op in ("loadVecGlobalCoord", "storeVecGlobalCoord"):
            at = f"coord{{(int){I(s.coordB)}, (int){I(s.coordD)}, (int){I(s.coordR)}, (int){I(s.coordC)}}}"
            return f"{ind}wave::{'load' if op == 'loadVecGlobalCoord' else 'store'}({I(s.dst)}, {I(s.src)}, {at});\n"
        if op == "storeGlobalAdd":
            tile = self.info[s.src]
            at = f"coord{{(int){I(s.coordB)}, (int){I(s.coordD)}, (int){I(s.coordR)} * {tile.rows}, (int){I(s.coordC)} * {tile.cols}}}"
            return f"{ind}wave::store_add({I(s.dst)}, {I(s.src)}, {at});\n"
        if op == "storeVecGlobalAdd":
            return f"{ind}wave::store_add({I(s.dst)}, {I(s.src)}, (int){I(s.offset)});\n"
        if op == "storeVecGlobalAddCoord":
            at = f"coord{{(int){I(s.coordB)}, (int){I(s.coordD)}, (int){I(s.coordR)}, (int){I(s.coordC)}}}"
            return f"{ind}wave::store_add({I(s.dst)}, {I(s.src)}, {at});\n"
        if op in ("cumsum", "cumprod"):
            f = "op_add" if op == "cumsum" else "op_mul"
            if s.axis == "Full":                         # the vector form: a running reduction along a register vector
                if self.kind(s.src) != "RV" or self.kind(s.dst) != "RV" or self.rv_layout[s.src] != "align":
                    raise UnsupportedStatement("a full scan runs along a per-row register vector")
                return f"{ind}wave::full_scan<{f}>({I(s.dst)}, {I(s.src)});\n"
            return f"{ind}wave::{s.axis.lower()}_scan<{f}>({I(s.dst)}, {I(s.src)});\n"
        if op == "loadScalarGlobal":
            return f"{ind}const auto {I(s.dst)} = {I(s.src)}.ptr[{I(s.offset)}];\n"
        if op == "storeScalarGlobal":
            return f"{ind}{I(s.dst)}.ptr[{I(s.offset)}] = {I(s.src)};\n"
        if op == "layoutDim":
            return f"{ind}const int {I(s.dst)} = {I(s.src)}.{s.axis.lower()}();\n"
        if op == "mma":
            b = self.streamed.get(s.b, s.b)              # a streamed operand is read from its LDS tile
            return f"{ind}wave::mma_{s.trans}({I(s.dst)}, {I(s.a)}, {I(b)}, {I(s.c)});\n"
        if op == "mm":
            return (f"{ind}wave::unary<op_zero>({I(s.dst)}, {I(s.dst)});\n"
                    f"{ind}wave::mma_{s.trans}({I(s.dst)}, {I(s.a)}, {I(s.b)}, {I(s.dst)});\n")
        if op == "unary":
            return f"{ind}wave::unary<{UNARY[s.args[0]]}>({I(s.dst)}, {I(s.src)});\n"
        if op == "binary":
            return f"{ind}wave::binary<{BINARY[s.args[0]]}>({I(s.dst)}, {I(s.a)}, {I(s.b)});\n"
        if op == "ternary":
            # FMA and FMAAxBtC are a * b + c, FMAAxCtB is a * c + b, element by element (the reference prints
            # warp::fma / fma_AxBtC / fma_AxCtB, Tyr/GPU/Codegen/AST.lean:196-206)
            x, y, z = (s.a, s.c, s.b) if s.args[0] == "FMAAxCtB" else (s.a, s.b, s.c)
            return f"{ind}wave::fma({I(s.dst)}, {I(x)}, {I(y)}, {I(z)});\n"
        if op in ("scalarMul", "scalarAdd"):
            f = "op_mul" if op == "scalarMul" else "op_add"
            return f"{ind}wave::scalar<{f}>({I(s.dst)}, {I(s.src)}, {_flt(s.scalar)});\n"
        if op == "broadcast":
            return f"{ind}wave::broadcast_{s.axis.lower()}({I(s.dst)}, {I(s.vec)});\n"
        if op == "binaryBroadcast":
            return f"{ind}wave::{s.axis.lower()}_broadcast<{BINARY[s.args[0]]}>({I(s.dst)}, {I(s.tile)}, {I(s.vec)});\n"
        if op in ("reduce", "reduceAccum"):
            tail = f", {I(s.accum)}" if op == "reduceAccum" else ""
            if s.axis == "Full":                         # every element of a vector or tile, left in every element of dst
                if self.kind(s.dst) != "RV" or (op == "reduceAccum" and self.kind(s.src) != "RV"):
                    raise UnsupportedStatement("a full reduction leaves its result in a register vector")
                return f"{ind}wave::full_reduce<{REDUCE[s.args[0]]}>({I(s.dst)}, {I(s.src)}{tail});\n"
            return f"{ind}wave::{s.axis.lower()}_reduce<{REDUCE[s.args[0]]}>({I(s.dst)}, {I(s.src)}{tail});\n"
        if op == "outer":
            return f"{ind}wave::outer({I(s.dst)}, {I(s.a)}, {I(s.b)});\n"
        if op == "transpose":
            t, d = self.info[s.src], self.info[s.dst]
            if s.dst == s.src and t.rows != t.cols:
                raise UnsupportedStatement("an in-place transpose needs a square tile")
            if t.layout == d.layout:     # same layout kind on both sides: the data really moves, through LDS
                return (f"{ind}{{\n{ind}  __shared__ st<{_cpp_type(t.dtype)}, {t.rows}, {t.cols}> {I(s.dst)}_tr;\n"
                        f"{ind}  wave::transpose({I(s.dst)}, {I(s.src)}, {I(s.dst)}_tr);\n{ind}}}\n")
            return f"{ind}wave::transpose({I(s.dst)}, {I(s.src)});\n"
        if op == "swapLayout":
            t = self.info[s.src]
            return (f"{ind}{{\n{ind}  __shared__ st<{_cpp_type(t.dtype)}, {t.rows}, {t.cols}> {I(s.dst)}_swap;\n"
                    f"{ind}  wave::swap_layout({I(s.dst)}, {I(s.src)}, {I(s.dst)}_swap);\n{ind}}}\n")
        if op == "convert":
            return f"{ind}wave::convert({I(s.dst)}, {I(s.src)});\n"
        if op == "mask":
            tag = s.args[0]
            if tag[0] == "UpperRightFill":
                fill = _flt(0.0 if s.fillVal is None else s.fillVal)
                return f"{ind}wave::mask_upper_right({I(s.dst)}, {I(s.src)}, {fill}, {tag[1]}, {tag[2]});\n"
            if tag[0] not in MASK:
                raise UnsupportedStatement(f"mask {tag[0]} has no gfx950 lowering yet")
            fill = _flt(0.0 if s.fillVal is None else s.fillVal)
            d = f", {tag[1]}" if len(tag) > 1 else ""
            return f"{ind}wave::mask<{MASK[tag[0]]}>({I(s.dst)}, {I(s.src)}, {fill}{d});\n"
        if op == "sliceRows":
            return f"{ind}wave::slice_rows<{s.startRow}>({I(s.dst)}, {I(s.src)});\n"
        if op == "sliceCols":
            return f"{ind}wave::slice_cols<{s.startCol}>({I(s.dst)}, {I(s.src)});\n"
        if op == "concatCols":
            return f"{ind}wave::concat_cols({I(s.dst)}, {I(s.left)}, {I(s.right)});\n"
        if op == "sync":
            return f"{ind}wave::sync();\n"
        if op in ("forLoop", "forLoopVal"):
            hi = f"{s.hi}" if op == "forLoop" else f"(int){I(s.hi)}"
            if self.group:                               # what the back edge may bring in, to a fixed point
                entry = set(self.dirty)
                while True:
                    end = self._dirty_after(s.body, entry) | entry
                    if end == entry:
                        break
                    entry = end
                self.dirty = set(entry)
            pre = self.prefetchable(s) if self.prefetch_global_loads else []
            if pre:
                return self.prefetched_loop(s, hi, pre, ind)
            return (f"{ind}for (int {I(s.v)} = {s.lo}; {I(s.v)} < {hi}; ++{I(s.v)}) {{\n" + self.body(s.body, ind + "  ") +
                    f"{ind}}}\n")
        if op == "ifStmt":
            out = f"{ind}if ({I(s.cond)}) {{\n" + self.body(s.thenBody, ind + "  ") + f"{ind}}}"
            if s.elseBody:
                out += " else {\n" + self.body(s.elseBody, ind + "  ") + f"{ind}}}"
            return out + "\n"
        if op == "comment":
            return f"{ind}// {s.text}\n"
        if op == "getBlockIdx":
            return f"{ind}const int {I(s.dst)} = blockIdx.{'xyz'[s.axis]};\n"
        if op == "getThreadIdx":
            return f"{ind}const int {I(s.dst)} = threadIdx.{'xyz'[s.axis]};\n"
        if op == "constInt":
            return f"{ind}const int {I(s.dst)} = {s.value};\n"
        if op == "constFloat":
            return f"{ind}const float {I(s.dst)} = {_flt(s.value)};\n"
        if op == "scalarUnary":
            e = f"-{I(s.src)}" if s.args[0] == "Neg" else f"__expf((float){I(s.src)})"
            return f"{ind}const auto {I(s.dst)} = {e};\n"
        if op == "scalarCompare":
            c = {"Eq": "==", "Lt": "<", "Le": "<=", "Gt": ">", "Ge": ">="}[s.args[0]]
            return f"{ind}const bool {I(s.dst)} = {I(s.a)} {c} {I(s.b)};\n"
        if op == "scalarBinary":
            o = s.args[0]
            if o in ("Min", "Max"):
                e = f"({I(s.a)} {'<' if o == 'Min' else '>'} {I(s.b)} ? {I(s.a)} : {I(s.b)})"
            else:
                sym = {"Add": "+", "Sub": "-", "Mul": "*", "Div": "/", "Mod": "%"}[o]
                e = f"{I(s.a)} {sym} {I(s.b)}"
            return f"{ind}const auto {I(s.dst)} = {e};\n"
        if op == "scalarSelect":
            return f"{ind}const auto {I(s.dst)} = {I(s.cond)} ? {I(s.ifTrue)} : {I(s.ifFalse)};\n"
        if op == "vecIota":
            return f"{ind}wave::iota({I(s.dst)}, {_flt(s.start)}, {_flt(s.step)});\n"
        if op == "vecFillScalar":
            return f"{ind}wave::fill({I(s.dst)}, (float){I(s.scalar)});\n"
        if op == "raw":
            return f"{ind}{s.code}\n"
        raise UnsupportedStatement(op)

    # ------------------------------------------------------------------ loops with prefetched tiles
    def prefetchable(self, loop: Stmt):
        """The leading loadGlobal statements of a loop body whose source and coordinates are the loop
        variable or values defined outside the loop.  Their global reads can be issued one iteration
        ahead (into registers) when nothing in the loop writes global memory."""
        inner = list(walk(loop.body))
        if any(t.op.startswith("store") and "Global" in t.op for t in inner):
            return []
        defined = {loop.v}
        for t in inner:
            for f in ("dst", "v"):
                x = getattr(t, f, None)
                if isinstance(x, VarId):
                    defined.add(x)
        out = []
        for t in loop.body:
            if t.op == "comment" or self._registers_only(t):
                continue                                 # declarations and register work in front of the loads stay where they are
            if t.op != "loadGlobal" or id(t) in self.barrier_before:
                break
            free = all(c == loop.v or c not in defined for c in (t.coordB, t.coordD, t.coordR, t.coordC))
            if not free or t.src in defined:
                break
            out.append(t)
        # a tile loaded twice in the body, or written by another statement, keeps the plain form
        written = [getattr(t, "dst", None) for t in inner if t not in out]
        out = [t for t in out if t.dst not in written and sum(1 for u in out if u.dst == t.dst) == 1]
        if self.group:                                   # the waves share a tile's 16-byte pieces evenly, or not at all
            def even(t):
                d = self.info[t.dst]
                return (d.rows * d.cols * _DTYPE_BYTES[d.dtype] // 16) % (64 * self.waves) == 0
            if not all(even(t) for t in out):
                return []
        return out

    def _registers_only(self, t: Stmt) -> bool:
        """A statement that touches register tiles / vectors and compile-time values only (no LDS, no global memory,
        no control flow)."""
        if t.op in ("forLoop", "forLoopVal", "ifStmt", "sync", "raw", "transpose", "swapLayout") or t.op in NVIDIA_ONLY:
            return False
        if t.op not in ("declRT", "declRV", "unary", "binary", "ternary", "scalarMul", "scalarAdd", "convert", "broadcast",
                        "binaryBroadcast", "vecFillScalar", "vecIota", "constInt", "constFloat"):
            return False
        return all(self.kind(a) in ("RT", "RV", "scalar") for a in t.args if isinstance(a, VarId))

    def prefetched_loop(self, loop: Stmt, hi: str, pre, ind: str) -> str:
        I = lambda v: v.ident
        frag = {id(t): f"{I(t.dst)}_next" for t in pre}

        def request(t, ind2):
            tile = self.info[t.dst]
            at = (f"coord{{(int){I(t.coordB)}, (int){I(t.coordD)}, (int){I(t.coordR)} * {tile.rows}, "
                  f"(int){I(t.coordC)} * {tile.cols}}}")
            if self.group:
                return f"{ind2}wave::gload_part({frag[id(t)]}, {I(t.src)}, {at}, tyr_wave);\n"
            return f"{ind2}wave::gload({frag[id(t)]}, {I(t.src)}, {at});\n"

        out = f"{ind}// the global tiles of iteration i+1 are requested while iteration i computes\n"
        for t in pre:
            tile = self.info[t.dst]
            if self.group:
                out += f"{ind}wave::gfrag_part<{_cpp_type(tile.dtype)}, {tile.rows}, {tile.cols}, {self.waves}> {frag[id(t)]};\n"
            else:
                out += f"{ind}wave::gfrag<{_cpp_type(tile.dtype)}, {tile.rows}, {tile.cols}> {frag[id(t)]};\n"
        out += f"{ind}if ({loop.lo} < {hi}) {{\n{ind}  const int {I(loop.v)} = {loop.lo};\n"
        out += "".join(request(t, ind + "  ") for t in pre) + f"{ind}}}\n"
        out += f"{ind}for (int {I(loop.v)} = {loop.lo}; {I(loop.v)} < {hi}; ++{I(loop.v)}) {{\n"
        ind2 = ind + "  "
        nxt = (f"{ind2}if ({I(loop.v)} + 1 < {hi}) {{\n{ind2}  const int {I(loop.v)}_n = {I(loop.v)} + 1;\n"
               f"{ind2}  {{\n{ind2}    const int {I(loop.v)} = {I(loop.v)}_n;\n" +
               "".join(request(t, ind2 + "    ") for t in pre) + f"{ind2}  }}\n{ind2}}}\n")
        placed = False
        remaining = len(pre)
        for t in self.fused(loop.body):
            if id(t) in frag:
                if id(t) in self.barrier_before:
                    out += f"{ind2}wave::sync();  // inserted: a shared tile is overwritten below after other waves read it\n"
                    self.dirty = set()
                if self.group:
                    out += f"{ind2}wave::sstore_part({I(t.dst)}, {frag[id(t)]}, tyr_wave);\n"
                    self.dirty.add(t.dst)
                else:
                    out += f"{ind2}wave::sstore({I(t.dst)}, {frag[id(t)]});\n"
                remaining -= 1
                continue
            out += self.one(t, ind2)
            if not placed and remaining == 0 and t.op == "sync":
                out += nxt
                placed = True
        if not placed:
            out += nxt
        return out + f"{ind}}}\n"

    def one(self, s: Stmt, ind: str) -> str:
        """A statement with the barriers it needs in front of it."""
        out = ""
        if id(s) in self.barrier_before:
            out += f"{ind}wave::sync();  // inserted: a shared tile is overwritten below after other waves read it\n"
            self.dirty = set()
        if self.group:
            reads, writes = self._group_rw(s)
            if reads & self.dirty:
                out += f"{ind}wave::sync();  // inserted: the other waves' shares of a shared tile are read below\n"
                self.dirty = set()
            if s.op == "sync":
                self.dirty = set()
            out += self.stmt(s, ind)
            if s.op not in ("forLoop", "forLoopVal", "ifStmt"):
                self.dirty |= writes
        else:
            out += self.stmt(s, ind)
        return out

    def body(self, stmts, ind: str) -> str:
        return "".join(self.one(s, ind) for s in self.fused(stmts))

    # ------------------------------------------------------------------ recognised statement sequences
    def fused(self, stmts):
        """The statement list with every occurrence of the online-softmax step (the expansion of the reference's
        `onlineSoftmax` macro, Macros.lean:121-147, with the score scaling in front of it if there is one) replaced by one
        call of `wave::online_softmax`.  Only register tiles and vectors are involved, so no barrier analysis refers to
        the statements that disappear."""
        if not self.fuse_online_softmax:
            return list(stmts)
        L, out, i = list(stmts), [], 0
        while i < len(L):
            m = self._match_online_softmax(L, i)
            if m is None:
                out.append(L[i])
                i += 1
            else:
                out.append(m[0])
                i = m[1]
        return out

    def _match_online_softmax(self, L, i):
        def nxt(j):                                      # next statement that is not a comment
            while j < len(L) and L[j].op == "comment":
                j += 1
            return j
        c, j = 1.0, nxt(i)
        if j < len(L) and L[j].op == "scalarMul" and L[j].dst == L[j].src and L[j].scalar > 0:
            c, S, j = L[j].scalar, L[j].dst, nxt(j + 1)
        else:
            S = None
        got = []
        for _ in range(9):
            if j >= len(L):
                return None
            got.append(L[j])
            j = nxt(j + 1)
        s1, s2, s3, s4, s5, s6, s7, s8, s9 = got
        try:
            ok = (s1.op == "unary" and s1.args[0] == "Copy" and
                  s2.op == "reduceAccum" and s2.args[0] == "Max" and s2.axis == "Row" and s2.dst == s2.accum == s1.src and
                  (S is None or s2.src == S) and
                  s3.op == "binary" and s3.args[0] == "Sub" and s3.a == s1.dst and s3.b == s2.dst and
                  s4.op == "unary" and s4.args[0] == "Exp" and s4.dst == s4.src == s3.dst and
                  s5.op == "binaryBroadcast" and s5.args[0] == "Mul" and s5.axis == "Col" and s5.dst == s5.tile and s5.vec == s3.dst and
                  s6.op == "binary" and s6.args[0] == "Mul" and s6.dst == s6.a and s6.b == s3.dst and
                  s7.op == "binaryBroadcast" and s7.args[0] == "Sub" and s7.axis == "Col" and s7.dst == s7.tile == s2.src and s7.vec == s2.dst and
                  s8.op == "unary" and s8.args[0] == "Exp" and s8.dst == s8.src == s2.src and
                  s9.op == "reduceAccum" and s9.args[0] == "Sum" and s9.axis == "Row" and s9.dst == s9.accum == s6.dst and s9.src == s2.src)
        except AttributeError:
            return None
        if not ok:
            return None
        S, O, mx, sm, prev, scl = s2.src, s5.dst, s2.dst, s6.dst, s1.dst, s3.dst
        if len({S, O}) != 2 or len({mx, sm, prev, scl}) != 4:
            return None
        for t in (S, O):
            d = self.info.get(t)
            if d is None or d.op != "declRT" or d.dtype != "Float32" or d.layout != "Row" or t in self.streamed:
                return None
        for v in (mx, sm, prev, scl):
            d = self.info.get(v)
            if d is None or d.op != "declRV" or d.dtype != "Float32" or self.rv_layout.get(v) != "align":
                return None
        if len({(v in self.split) for v in (S, O, mx, sm, prev, scl)}) != 1:
            return None
        from .ir import stmt as mk
        code = (f"wave::online_softmax({S.ident}, {O.ident}, {mx.ident}, {sm.ident}, {prev.ident}, {scl.ident}, {_flt(c)});"
                f"  // the online-softmax step{' with its score scale' if c != 1.0 else ''}, fused")
        return mk("raw", code), j

    # ------------------------------------------------------------------ wave groups: who reads whose share
    def _group_rw(self, s: Stmt):
        """(LDS objects the statement reads in full, LDS objects it leaves written in per-wave shares)."""
        if s.op in ("forLoop", "forLoopVal"):
            return set(), set()                          # handled when the loop is emitted
        if s.op == "ifStmt":                             # a barrier cannot sit inside a conditional
            r, w = set(), set()
            for t in walk(s.thenBody + s.elseBody):
                a, b = self._group_rw(t)
                r |= a
                w |= b
            return r, w
        if s.op == "load":
            return (set() if s.dst in self.streamed else {s.src}), set()
        if s.op == "store":
            return set(), ({s.dst} if s.src in self.split else set())
        if s.op == "loadGlobal":
            return set(), {s.dst}
        if s.op in ("storeGlobal", "storeGlobalAdd", "storeVecGlobal", "storeVecGlobalCoord", "storeVecGlobalAdd",
                    "storeVecGlobalAddCoord"):
            return {s.src}, set()
        if s.op == "mma" and s.b in self.streamed:
            return {self.streamed[s.b]}, set()
        return set(), set()

    def _dirty_after(self, stmts, dirty: set) -> set:
        dirty = set(dirty)
        for s in stmts:
            if id(s) in self.barrier_before or s.op == "sync":
                dirty = set()
            if s.op in ("forLoop", "forLoopVal"):
                entry = set(dirty)
                while True:
                    end = self._dirty_after(s.body, entry) | entry
                    if end == entry:
                        break
                    entry = end
                dirty = self._dirty_after(s.body, entry)
                continue
            reads, writes = self._group_rw(s)
            if reads & dirty:
                dirty = set()
            dirty |= writes
        return dirty

    # ------------------------------------------------------------------ kernel + launchers
    def param_decls(self):
        """(kernel parameter text, VarId) in signature order: the k-th parameter is the k-th
        declGPtr / declKVal statement."""
        decls = [s for s in self.k.body if s.op in ("declGPtr", "declKVal")]
        assert len(decls) == len(self.k.params), "every parameter needs its declGPtr / declKVal statement"
        out = []
        for p, d in zip(self.k.params, decls):
            if p.isPointer:
                out.append((f"gl<{_cpp_type(p.dtype)}> {d.v.ident}", d.v, p))
            else:
                out.append((f"{K_SCALAR_TYPES[p.scalarTy]} {d.v.ident}", d.v, p))
        return out

    def kernel_text(self) -> str:
        sig = ", ".join(t for t, _, _ in self.param_decls())
        pool = ""
        if self.lds:
            decl = {t.v: t for t in walk(self.k.body) if t.op == "declST"}
            total = max(off + st_bytes(decl[v]) for v, off in self.lds.items())
            pool = (f"  // LDS tiles whose live ranges do not intersect share these bytes\n"
                    f"  __shared__ __attribute__((aligned(16))) unsigned char tyr_lds_pool[{total}];\n")
        head = ""
        if self.group:
            head = (f"  // run by a group of {self.waves} waves: row-tied register tiles are cut into {self.waves} row slices\n"
                    f"  const int tyr_wave = wave::index();\n")
        self.dirty = set()
        bounds = f"{64 * self.max_waves}, {self.min_blocks}" if self.min_blocks > 1 else f"{64 * self.max_waves}"
        return (f"__global__ __launch_bounds__({bounds}) void {self.k.name}({sig}) {{\n" + pool + head +
                self.body(self.k.body, "  ") + "}\n")

    def launcher_signature(self) -> str:
        cparams = []
        for _, _, p in self.param_decls():
            if p.isPointer:
                cparams += [f"void* {p.name}", f"const int64_t* {p.name}_shape", f"int {p.name}_ndim"]
            else:
                cparams.append(f"{K_SCALAR_TYPES[p.scalarTy]} {p.name}")
        cparams += ["uint64_t grid_x", "uint64_t grid_y", "uint64_t grid_z", "uint64_t block_x", "uint64_t block_y",
                    "uint64_t block_z", "uint64_t shared_mem", "void* stream"]
        return f"int tyr_launch_{self.k.name}({', '.join(cparams)})"

    def launcher_text(self) -> str:
        name, decls = self.k.name, self.param_decls()
        cparams, setup, args = [], [], []
        for i, (_, v, p) in enumerate(decls):
            if p.isPointer:
                cparams += [f"void* {p.name}", f"const int64_t* {p.name}_shape", f"int {p.name}_ndim"]
                setup.append(
                    f"  if ({p.name} == nullptr || {p.name}_ndim < 0 || {p.name}_ndim > 4) return -2;\n"
                    f"  int s{i}[4] = {{1, 1, 1, 1}};\n"
                    f"  for (int i = 0; i < {p.name}_ndim; ++i) s{i}[4 - {p.name}_ndim + i] = (int){p.name}_shape[i];\n"
                    f"  gl<{_cpp_type(p.dtype)}> g{i}{{static_cast<{_cpp_type(p.dtype)}*>({p.name}), s{i}[0], s{i}[1], s{i}[2], s{i}[3]}};\n")
                args.append(f"g{i}")
            else:
                cparams.append(f"{K_SCALAR_TYPES[p.scalarTy]} {p.name}")
                args.append(p.name)
        cparams += ["uint64_t grid_x", "uint64_t grid_y", "uint64_t grid_z", "uint64_t block_x", "uint64_t block_y",
                    "uint64_t block_z", "uint64_t shared_mem", "void* stream"]
        return (
            f"// C ABI: tensors as (device pointer, shape, rank <= 4), then the kernel's scalars, then the launch\n"
            f"// geometry of the reference launcher (Tyr/GPU/Codegen/Attribute.lean:344-386).  A 32-thread warp of\n"
            f"// the requested block becomes one 64-lane wave.  Returns 0, -2 (bad argument) or -1 (launch error).\n"
            f"extern \"C\" int tyr_launch_{name}({', '.join(cparams)}) {{\n" + "".join(setup) +
            f"  const uint64_t threads = block_x * block_y * block_z;\n"
            f"  if (threads == 0 || grid_x * grid_y * grid_z == 0) return -2;\n" +
            (f"  // Every warp of the reference's block repeats the whole tile program, so the block shape does not change the\n"
             f"  // result; here the program is cut into the row slices of a group of exactly {self.waves} waves, whatever was asked for.\n"
             f"  const unsigned waves = {self.waves};\n"
             if self.group else
             f"  const unsigned waves = (unsigned)((threads + 31) / 32);\n"
             f"  if (waves > {self.max_waves}) return -2;\n") +
            f"  hipLaunchKernelGGL({name}, dim3((unsigned)grid_x, (unsigned)grid_y, (unsigned)grid_z), dim3(64 * waves), "
            f"(size_t)shared_mem, static_cast<hipStream_t>(stream), {', '.join(args)});\n"
            f"  return hipGetLastError() == hipSuccess ? 0 : -1;\n}}\n")

    def lean_launcher_text(self) -> str:
        """`lean_launch_<kernel>` with the reference's signature, checks and messages
        (Attribute.lean:318-386), over the C-ABI launcher above."""
        name, decls = self.k.name, self.param_decls()
        lparams, setup, args = [], [], []
        for i, (_, v, p) in enumerate(decls):
            if p.isPointer:
                lparams.append(f"b_lean_obj_arg {p.name}")
                setup.append(
                    f"  auto t{i} = borrowTensor({p.name});\n"
                    f"  if (!t{i}.is_cuda()) return tyr_dsl_io_error(\"{p.name} must be a CUDA tensor\");\n"
                    f"  if (!t{i}.is_contiguous()) return tyr_dsl_io_error(\"{p.name} must be contiguous\");\n"
                    f"  if (t{i}.dim() > 4) return tyr_dsl_io_error(\"{p.name} must have dim <= 4\");\n"
                    f"  int64_t shape{i}[4] = {{1, 1, 1, 1}};\n"
                    f"  for (int i = 0; i < (int)t{i}.dim(); ++i) shape{i}[i] = t{i}.size(i);\n")
                args += [f"t{i}.data_ptr()", f"shape{i}", f"(int)t{i}.dim()"]
            else:
                lparams.append(f"{K_SCALAR_TYPES[p.scalarTy]} {p.name}")
                args.append(p.name)
        lparams += ["uint64_t grid_x", "uint64_t grid_y", "uint64_t grid_z", "uint64_t block_x", "uint64_t block_y",
                    "uint64_t block_z", "uint64_t shared_mem", "uint64_t stream", "lean_object* /* world */"]
        args += ["grid_x", "grid_y", "grid_z", "block_x", "block_y", "block_z", "shared_mem",
                 "reinterpret_cast<void*>(stream)"]
        return (f"extern \"C\" lean_object* lean_launch_{name}({', '.join(lparams)}) {{\n  try {{\n" +
                "".join("  " + l + "\n" for l in "".join(setup).splitlines()) +
                f"    const int rc = tyr_launch_{name}({', '.join(args)});\n"
                f"    if (rc == -2) return tyr_dsl_io_error(\"invalid launch arguments for {name}\");\n"
                f"    if (rc != 0) return tyr_dsl_io_error(hipGetErrorString(hipGetLastError()));\n"
                f"    return lean_io_result_mk_ok(lean_box(0));\n"
                f"  }} catch (const std::exception& e) {{\n    return tyr_dsl_io_error(e.what());\n  }}\n}}\n")


PREAMBLE = """// Emitted from the tile DSL for gfx950; do not edit.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "tile/tyr_tile.hpp"

using namespace tyr::tile;

"""

LEAN_PREAMBLE = """#if defined(__has_include)
#if __has_include(<lean/lean.h>) && __has_include(<torch/torch.h>)
#define TYR_HAVE_LEAN 1
#endif
#endif
#ifdef TYR_HAVE_LEAN
#include <lean/lean.h>
#include <torch/torch.h>
torch::Tensor borrowTensor(b_lean_obj_arg o);   // cc/src/tyr.cpp:127-148
static lean_object* tyr_dsl_io_error(const char* msg) {
  return lean_io_result_mk_error(lean_mk_io_user_error(lean_mk_string(msg)));
}
"""


def emit_header(kernels: List[Kernel], cites: Dict[str, str]) -> str:
    """C declarations of the launchers of `kernels`; `cites` maps a kernel name to the reference
    definition whose generated `lean_launch_<kernel>` (Attribute.lean:344-386) the entry point stands in for."""
    out = ("/* C ABI of the tile programs emitted for gfx950 (libtyr_dsl.so).  Generated by tyr_amd.dsl; do not edit.\n"
           " *\n"
           " * Every entry point replaces the launcher the reference generates for the same kernel,\n"
           " * `lean_launch_<kernel>` (Tyr/GPU/Codegen/Attribute.lean:344-386): tensors arrive as (device pointer,\n"
           " * shape, rank <= 4; right-aligned into batch, depth, rows, cols as the reference does,\n"
           " * Attribute.lean:337-342), then the kernel's scalar parameters, then grid, block, dynamic shared\n"
           " * memory and the stream.  A 32-thread warp of the requested block is run as one 64-lane wave.\n"
           " * Returns 0 on success, -2 for an invalid argument, -1 if the launch failed. */\n"
           "#ifndef TYR_DSL_KERNELS_H\n#define TYR_DSL_KERNELS_H\n\n#include <stdint.h>\n\n"
           "#ifdef __cplusplus\nextern \"C\" {\n#endif\n\n")
    for k in kernels:
        out += f"/* {cites[k.name]} */\n{_Emitter(k).launcher_signature()};\n\n"
    return out + "#ifdef __cplusplus\n}\n#endif\n\n#endif /* TYR_DSL_KERNELS_H */\n"


def emit_kernel(kernel: Kernel, hazard_barriers: bool = True, prefetch_global_loads: bool = True,
                share_lds: bool = True, fuse_online_softmax: bool = True) -> str:
    """Device code of one kernel (no includes)."""
    return _Emitter(kernel, hazard_barriers=hazard_barriers, prefetch_global_loads=prefetch_global_loads,
                    share_lds=share_lds, fuse_online_softmax=fuse_online_softmax).kernel_text()


def emit_translation_unit(kernels: List[Kernel]) -> str:
    """One .hip file: every kernel, its C-ABI launcher, and (where Lean headers exist) its
    `lean_launch_*` wrapper."""
    ems = [_Emitter(k) for k in kernels]
    out = PREAMBLE
    for e in ems:
        out += e.kernel_text() + "\n" + e.launcher_text() + "\n"
    out += LEAN_PREAMBLE + "".join(e.lean_launcher_text() + "\n" for e in ems) + "#endif  // TYR_HAVE_LEAN\n"
    return out
