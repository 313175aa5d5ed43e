/-
  Tyr.GPU.GFX950 — entry points of the MI355X (gfx950 / CDNA4) kernel library.

  These are plain `@[extern]` opaques in the style of `Tyr/Torch.lean:1058-1082`
  (`scaledDotProductAttentionGQA`), not `@[gpu_kernel]` DSL kernels: the kernels behind
  them are hand-written HIP, so no `GpuArch` constructor is involved and none of the
  exhaustive matches on `GpuArch` change.  Shapes are carried in the types; the implicit
  `UInt64` binders reach the C side first, unboxed, in binder order.

  Unlike the generated `X.launch … : IO Unit` launchers (`Tyr/GPU/Codegen/Attribute.lean:390-437`),
  which mutate caller-allocated outputs behind Lean's back, these return freshly allocated
  tensors in `IO`.

  C side: `tyr_amd/csrc/lean_shim.cpp` (wrappers) over `include/tyr_hip.h` (C ABI).
-/
import Tyr.Basic
import Tyr.GPU.Codegen.TileTypes

namespace Tyr.GPU.GFX950

open torch
open Tyr.GPU.Codegen (CudaStream)

/-- Capabilities of the one target this library is built for. Nothing matches on it. -/
structure Capabilities where
  arch : String := "gfx950"
  waveSize : Nat := 64
  computeUnits : Nat := 256
  ldsBytesPerCU : Nat := 163840
  /-- dense bf16 MFMA tile shapes used by the kernels (M, N, K) -/
  mfmaBf16 : List (Nat × Nat × Nat) := [(32, 32, 16), (16, 16, 32)]
  /-- dense FP8 (OCP E4M3) MFMA tile shape -/
  mfmaFp8 : List (Nat × Nat × Nat) := [(32, 32, 64)]
  fp8Format : String := "OCP e4m3fn (bias 7, max 448, no inf)"
  deriving Repr

def capabilities : Capabilities := {}

/-- Flash-attention forward. `q k v : bf16 [B,H,N,D]`, `D ∈ {64,128}`.
    Returns `(O : bf16 [B,H,N,D], LSE : f32 [B,H,N])` with `LSE = ln Σ_j exp(scale · qᵢ·kⱼ)`.
    GPU twin of `nn.scaled_dot_product_attention` (`Tyr/Torch.lean:665-671`). -/
@[extern "lean_tyr_gpu_flash_attn_fwd"]
opaque flashAttnFwd {B H N D : UInt64} (q k v : @& T #[B, H, N, D]) (causal : Bool) (scale : Float)
    (stream : CudaStream) : IO (T #[B, H, N, D] × T #[B, H, N])

/-- Flash-attention forward with grouped queries (`k v` carry `Hkv` heads, query head `h` reads kv head
    `h / (Hq/Hkv)`), a causal sliding window (`window = 0`: none) and per-sequence key lengths
    (`kvLens : int32 [B]`, keys at or beyond them are masked). GPU twin of `nn.scaledDotProductAttentionGQA`,
    `…GQAWindow` and (for prefix padding masks) `…GQAMask` (`cc/src/tyr.cpp:3913-4095`; callers
    `Tyr/Model/Qwen/Attention.lean:138,274`, `Tyr/Model/Qwen3TTS/SpeechTokenizer.lean:591`). -/
@[extern "lean_tyr_gpu_flash_attn_fwd_gqa"]
opaque flashAttnFwdGQA {B Hq Hkv N D : UInt64} (q : @& T #[B, Hq, N, D]) (k v : @& T #[B, Hkv, N, D])
    (kvLens : @& T #[B]) (causal : Bool) (window : UInt64) (scale : Float) (stream : CudaStream)
    : IO (T #[B, Hq, N, D] × T #[B, Hq, N])

/-- `flashAttnFwdGQA` for a batch whose sequences all have `N` keys: no length tensor, and with `window = 0`
    the launch takes the kernel instantiation that carries no length or window instructions (the one
    `flashAttnFwd` runs), which is what a model's ordinary prefill wants (`Tyr/Model/Qwen/Attention.lean:138`). -/
@[extern "lean_tyr_gpu_flash_attn_fwd_gqa_full"]
opaque flashAttnFwdGQAFull {B Hq Hkv N D : UInt64} (q : @& T #[B, Hq, N, D]) (k v : @& T #[B, Hkv, N, D])
    (causal : Bool) (window : UInt64) (scale : Float) (stream : CudaStream)
    : IO (T #[B, Hq, N, D] × T #[B, Hq, N])

/-- Flash-attention backward. `o` and `lse` are the results of `flashAttnFwd` for the same
    `q k v causal scale`; `dO` is the upstream gradient. Returns `(dQ, dK, dV)`, bf16, final
    (no per-tile partials to reduce on the host). Replaces `tkMhaH100BwdPrep2Block` +
    `tkMhaH100Bwd2BlockPartials` (`Tyr/GPU/Kernels/MhaH100.lean:197-344`) for any `B H N`;
    the values are autograd's for `nn.scaled_dot_product_attention`
    (`Examples/GPU/RunMhaH100.lean:56-64`). -/
@[extern "lean_tyr_gpu_flash_attn_bwd"]
opaque flashAttnBwd {B H N D : UInt64} (q k v o : @& T #[B, H, N, D]) (lse : @& T #[B, H, N])
    (dO : @& T #[B, H, N, D]) (causal : Bool) (scale : Float) (stream : CudaStream)
    : IO (T #[B, H, N, D] × T #[B, H, N, D] × T #[B, H, N, D])

/-- Backward of `flashAttnFwdGQA` (same `q k v kvLens causal window scale`; `o lse` its results).
    Returns `(dQ : [B,Hq,N,D], dK, dV : [B,Hkv,N,D])`; `dK dV` are summed over the query heads that read
    each kv head, which is the gradient of the reference's `repeat_interleave` (`cc/src/tyr.cpp:3930-3936`). -/
@[extern "lean_tyr_gpu_flash_attn_bwd_gqa"]
opaque flashAttnBwdGQA {B Hq Hkv N D : UInt64} (q : @& T #[B, Hq, N, D]) (k v : @& T #[B, Hkv, N, D])
    (o : @& T #[B, Hq, N, D]) (lse : @& T #[B, Hq, N]) (dO : @& T #[B, Hq, N, D]) (kvLens : @& T #[B])
    (causal : Bool) (window : UInt64) (scale : Float) (stream : CudaStream)
    : IO (T #[B, Hq, N, D] × T #[B, Hkv, N, D] × T #[B, Hkv, N, D])

/-- Backward of `flashAttnFwdGQAFull`. -/
@[extern "lean_tyr_gpu_flash_attn_bwd_gqa_full"]
opaque flashAttnBwdGQAFull {B Hq Hkv N D : UInt64} (q : @& T #[B, Hq, N, D]) (k v : @& T #[B, Hkv, N, D])
    (o : @& T #[B, Hq, N, D]) (lse : @& T #[B, Hq, N]) (dO : @& T #[B, Hq, N, D])
    (causal : Bool) (window : UInt64) (scale : Float) (stream : CudaStream)
    : IO (T #[B, Hq, N, D] × T #[B, Hkv, N, D] × T #[B, Hkv, N, D])

/-- `flashAttnFwdGQA` with an arbitrary key mask instead of lengths: `keyMask : uint8 [B,N]`, key `j` of
    sequence `b` is visible iff `keyMask[b,j] ≠ 0` (and `j ≤ i` when `causal`). GPU twin of
    `nn.scaledDotProductAttentionGQAMask` (`cc/src/tyr.cpp:4019-4095`) for any mask, e.g. left padding;
    a row that sees no key gets `O = 0`, `LSE = -∞` where LibTorch returns NaN. -/
@[extern "lean_tyr_gpu_flash_attn_fwd_mask"]
opaque flashAttnFwdMask {B Hq Hkv N D : UInt64} (q : @& T #[B, Hq, N, D]) (k v : @& T #[B, Hkv, N, D])
    (keyMask : @& T #[B, N]) (causal : Bool) (scale : Float) (stream : CudaStream)
    : IO (T #[B, Hq, N, D] × T #[B, Hq, N])

/-- Backward of `flashAttnFwdMask` (same `q k v keyMask causal scale`; `o lse` its results): hidden keys
    receive `dK = dV = 0`, rows that saw no key `dQ = 0`. -/
@[extern "lean_tyr_gpu_flash_attn_bwd_mask"]
opaque flashAttnBwdMask {B Hq Hkv N D : UInt64} (q : @& T #[B, Hq, N, D]) (k v : @& T #[B, Hkv, N, D])
    (o : @& T #[B, Hq, N, D]) (lse : @& T #[B, Hq, N]) (dO : @& T #[B, Hq, N, D]) (keyMask : @& T #[B, N])
    (causal : Bool) (scale : Float) (stream : CudaStream)
    : IO (T #[B, Hq, N, D] × T #[B, Hkv, N, D] × T #[B, Hkv, N, D])

/-- GQA decode attention, one query token per sequence, split-KV with an LSE combine pass.
    `q : bf16 [B,Hq,1,D]`, `k v : bf16 [B,Hkv,L,D]` (contiguous cache), `D ∈ {64, 128}`,
    query head `h` reads kv head `h / (Hq/Hkv)`; `numSplits = 0` lets the library choose.
    GPU twin of `nn.scaledDotProductAttentionGQAQKV` with `is_causal = false`
    (`Tyr/Torch.lean:1070-1082`, caller `Tyr/Model/Qwen/Attention.lean:199-200`). -/
@[extern "lean_tyr_gpu_gqa_decode"]
opaque gqaDecode {B Hq Hkv L D : UInt64} (q : @& T #[B, Hq, 1, D]) (k v : @& T #[B, Hkv, L, D])
    (scale : Float) (numSplits : UInt64) (stream : CudaStream) : IO (T #[B, Hq, 1, D] × T #[B, Hq])

/-- `gqaDecode` with a per-sequence cache length (`kvLens : int32 [B]`, a padding mask over the cache
    tail) and a sliding window (`window = 0`: unbounded): sequence `b` attends to cache rows
    `[max 0 (kvLens[b] - window), kvLens[b])`. Decode-time form of `nn.scaledDotProductAttentionGQAMask` and
    `nn.scaledDotProductAttentionGQAWindow` (`cc/src/tyr.cpp:3953-4095`). -/
@[extern "lean_tyr_gpu_gqa_decode_varlen"]
opaque gqaDecodeVarlen {B Hq Hkv L D : UInt64} (q : @& T #[B, Hq, 1, D]) (k v : @& T #[B, Hkv, L, D])
    (kvLens : @& T #[B]) (window : UInt64) (scale : Float) (numSplits : UInt64) (stream : CudaStream)
    : IO (T #[B, Hq, 1, D] × T #[B, Hq])

/-- Decode step between the projections and `gqaDecode`: rotary embedding of the single-token `q` and
    `kNew` (`cos sin : f32 [1, D/2]`, the table row of position `pos`), then `kNew` (rotated) and `vNew`
    are written into row `pos` of the preallocated caches **in place**. Returns the rotated `q`.
    Fuses `rotary.applyRotaryEmb` ×2 and `data.sliceScatter` ×2 of `QwenAttention.forwardStep`
    (`Tyr/Model/Qwen/Attention.lean:172-196`); follow with `gqaDecode` over the first `pos+1` rows. -/
@[extern "lean_tyr_gpu_decode_rope_append"]
opaque decodeRopeAppend {B Hq Hkv L D : UInt64} (q : @& T #[B, Hq, 1, D]) (kNew vNew : @& T #[B, Hkv, 1, D])
    (cos sin : @& T #[1, D / 2]) (kCache vCache : @& T #[B, Hkv, L, D]) (pos : UInt64) (stream : CudaStream)
    : IO (T #[B, Hq, 1, D])

/-- Rotary embedding, `x : f32 | bf16 [B,S,H,D]`, `cos sin : f32 [S, D/2]`; GPU twin of
    `rotary.applyRotaryEmb` (`Tyr/Torch.lean:1044`, `cc/src/tyr.cpp:3837-3873`) and of the DSL kernel
    `rotaryFwd` (`Tyr/GPU/Kernels/Rotary.lean:13-66`). -/
@[extern "lean_tyr_gpu_rope_fwd"]
opaque applyRotaryEmb {B S H D : UInt64} (x : @& T #[B, S, H, D]) (cos sin : @& T #[S, D / 2])
    (stream : CudaStream) : IO (T #[B, S, H, D])

/-- Fused residual add + LayerNorm over the last axis, bf16: returns `(out, outResid)` with
    `outResid = x + residual`. Replaces `tkFusedLayerNormResidual1024`
    (`Tyr/GPU/Kernels/FusedLayerNorm.lean:28-140`) for any `rows` and `d ≤ 8192`, `d % 8 = 0`. -/
@[extern "lean_tyr_gpu_layernorm_residual"]
opaque fusedLayerNormResidual {rows d : UInt64} (x residual : @& T #[rows, d]) (weight bias : @& T #[d])
    (eps : Float) (stream : CudaStream) : IO (T #[rows, d] × T #[rows, d])

/-- Device copy; replaces `copy64x64` (`Tyr/GPU/Kernels/Copy.lean:16-27`) for any contiguous tensor. -/
@[extern "lean_tyr_gpu_copy"]
opaque copy {s : Shape} (input : @& T s) (stream : CudaStream) : IO (T s)

/-- `C = A · B`, bf16 operands, f32 accumulation, bf16 result; `b` is `K × N` row-major.
    GPU twin of `nn.mm` (`Tyr/Torch.lean:546`). -/
@[extern "lean_tyr_gpu_gemm_bf16"]
opaque gemmBf16 {M N K : UInt64} (a : @& T #[M, K]) (b : @& T #[K, N]) (stream : CudaStream)
    : IO (T #[M, N])

/-- `C = A · Bᵀ` with `b` stored `N × K` (the operand layout of `tiledAccumulator`,
    `Tyr/GPU/Kernels/GemmCommon.lean:22-56`). -/
@[extern "lean_tyr_gpu_gemm_bf16_nt"]
opaque gemmBf16NT {M N K : UInt64} (a : @& T #[M, K]) (b : @& T #[N, K]) (stream : CudaStream)
    : IO (T #[M, N])

/-- FP8 (e4m3fn) GEMM with per-tensor scales: `C = bf16 (scaleA · scaleB · (Aq · Bq))`.
    Counterpart of `gemmFp8E4M3Fwd` / `tkH100Fp8ScaledGemmFwd`
    (`Tyr/GPU/Kernels/PrecisionGemm.lean:97-115,178-189`). -/
@[extern "lean_tyr_gpu_gemm_fp8"]
opaque gemmFp8 {M N K : UInt64} (a : @& T #[M, K]) (b : @& T #[K, N]) (scaleA scaleB : Float)
    (stream : CudaStream) : IO (T #[M, N])

/-- Batched matmul of rank-3 operands in one launch: `C[i] = A[i] · B[i]`. GPU twin of `torch.matmul`
    (`lean_torch_matmul`, `cc/src/tyr.cpp:1565-1570`) for `[Bt, M, K] × [Bt, K, N]`. -/
@[extern "lean_tyr_gpu_matmul_bf16"]
opaque matmulBf16 {Bt M N K : UInt64} (a : @& T #[Bt, M, K]) (b : @& T #[Bt, K, N]) (stream : CudaStream)
    : IO (T #[Bt, M, N])

/-- FP8 GEMM with per-row and per-column f32 dequantisation scales and f32 output:
    `C[m,n] = rowScale[m] · colScale[n] · (Aq · Bq)[m,n]`, the epilogue of `tkH100Fp8ScaledGemmFwd`
    (`Tyr/GPU/Kernels/PrecisionGemm.lean:97-115`, `GemmCommon.lean:83-133`). -/
@[extern "lean_tyr_gpu_gemm_fp8_scaled"]
opaque gemmFp8Scaled {M N K : UInt64} (a : @& T #[M, K]) (b : @& T #[K, N]) (rowScale : @& T #[M])
    (colScale : @& T #[N]) (stream : CudaStream) : IO (T #[M, N])

/-- FP8 GEMM with E4M3 output (round to nearest even, saturating at ±448): `tkH100Fp8E4M3GemmFwd`
    (`Tyr/GPU/Kernels/PrecisionGemm.lean:78-89`). `scale` multiplies the f32 accumulators before the cast. -/
@[extern "lean_tyr_gpu_gemm_fp8_e4m3"]
opaque gemmFp8E4M3 {M N K : UInt64} (a : @& T #[M, K]) (b : @& T #[K, N]) (scale : Float)
    (stream : CudaStream) : IO (T #[M, N])

/-- `lossAndGradOut` of the attention train step (`Examples/GPU/RunMhaH100Train.lean:60-67`) as one pass:
    `loss = 0.5 · mean((out − target)²)` (an f32 scalar tensor) and `dO = bf16((out − target) / numel)`. -/
@[extern "lean_tyr_gpu_mse_loss_grad"]
opaque lossAndGradOut {s : Shape} (out target : @& T s) (stream : CudaStream) : IO (T #[] × T s)

/-- `sgdUpdate` (`Examples/GPU/RunMhaH100Train.lean:69-70`) fused with the bf16 cast of the next step (`:83-85`):
    returns `(param − f32(grad) · lr, bf16 of that)`; `param` f32, `grad` bf16, bit-identical to the LibTorch chain. -/
@[extern "lean_tyr_gpu_sgd_step"]
opaque sgdUpdate {s : Shape} (param grad : @& T s) (lr : Float) (stream : CudaStream) : IO (T s × T s)

end Tyr.GPU.GFX950
