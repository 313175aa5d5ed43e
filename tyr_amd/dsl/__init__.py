"""Tile DSL for gfx950: the reference's kernel IR and builder vocabulary (Tyr/GPU/Codegen) with a HIP
emitter in place of its CUDA one."""
from .builder import KernelBuilder  # noqa: F401
from .emit import LayoutConflict, UnsupportedStatement, emit_header, emit_kernel, emit_translation_unit, infer_rv_layouts  # noqa: F401
from .ir import KSTMT_FIELDS, KParam, Kernel, Stmt, VarId, stmt  # noqa: F401
