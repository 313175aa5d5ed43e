/*
 * tyr_hip.h -- C ABI of the gfx950 (MI355X) kernel library behind Tyr's GPU surface.
 *
 * Plain pointers and sizes only: no torch, no Lean types.  Every pointer is a
 * device pointer into HBM unless stated otherwise; every tensor is dense and
 * row-major ("contiguous") with the stated shape.  `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  Launches are asynchronous on
 * that stream; the caller synchronises, exactly as with the reference's
 * generated launchers (Tyr/GPU/Codegen/Attribute.lean:346-386: launch, then
 * cudaGetLastError, no synchronisation).
 *
 * All functions return TYR_HIP_OK (0) or a negative tyr_hip_status; they never
 * throw and never abort.  tyr_hip_strerror() gives the message a Lean wrapper
 * puts into `IO.userError` (the reference's convention,
 * Tyr/GPU/Codegen/Attribute.lean:334-336,380-384).
 *
 * bf16 tensors are uint16 bit patterns in memory; e4m3 tensors are OCP FP8
 * E4M3 ("e4m3fn": bias 7, max 448, no infinity) bytes.
 */
#ifndef TYR_HIP_H
#define TYR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tyr_hip_status {
    TYR_HIP_OK = 0,
    TYR_HIP_ERR_NULL_POINTER = -1,   /* a required pointer argument is NULL            */
    TYR_HIP_ERR_BAD_SHAPE = -2,      /* zero/negative/inconsistent extents             */
    TYR_HIP_ERR_UNSUPPORTED = -3,    /* valid request the kernels do not implement     */
    TYR_HIP_ERR_MISALIGNED = -4,     /* pointer or row pitch not 16-byte aligned       */
    TYR_HIP_ERR_WORKSPACE = -5,      /* workspace missing or too small                 */
    TYR_HIP_ERR_LAUNCH = -6,         /* HIP reported a launch error                    */
    TYR_HIP_ERR_NO_DEVICE = -7,      /* no gfx950 device / library built without HIP   */
    TYR_HIP_ERR_NOT_DEVICE_MEMORY = -8 /* tyr_hip_check_device_pointer: host pointer   */
} tyr_hip_status;

/* Message for a status code; static storage, never NULL. */
const char* tyr_hip_strerror(int status);

/* Library/ABI version (major*10000 + minor*100 + patch). */
int tyr_hip_version(void);

/* Fills the properties the harness prints next to every figure.  Any pointer may be NULL.
 * Returns TYR_HIP_ERR_NO_DEVICE when no GPU is visible. */
int tyr_hip_device_info(int device, char* name, size_t name_len, int* compute_units,
                        int* lds_bytes_per_cu, int* clock_mhz, size_t* hbm_bytes);

/* The "<p> must be a CUDA tensor" check of the reference's launcher
 * (Tyr/GPU/Codegen/Attribute.lean:334), for callers that hold raw pointers:
 * TYR_HIP_OK if `p` is device memory, TYR_HIP_ERR_NOT_DEVICE_MEMORY otherwise. */
int tyr_hip_check_device_pointer(const void* p);

/* ---------------------------------------------------------------------------
 * Flash-attention forward:  O = softmax(Q K^T * scale [+ causal mask]) V,
 * LSE[b,h,i] = ln sum_j exp(scale * q_i . k_j)   (natural log of the scaled scores).
 *
 * Replaces the reference's DSL attention forward kernels and their launchers
 * (Tyr/GPU/Kernels/MhaH100.lean:71-128 `tkFlashAttnFwd2BlockLse`,
 *  Tyr/GPU/Kernels/MhaH100LCF.lean:29-132 for D=128; launcher text
 *  Tyr/GPU/Codegen/Attribute.lean:346-386) and is the GPU twin of
 * `lean_torch_sdpa_4d` (cc/src/tyr.cpp:2563-2589).
 *
 *   q, k, v : bf16 [B, H, N, D]        o : bf16 [B, H, N, D]
 *   lse     : f32  [B, H, N]  (may be NULL: not written)
 *   causal  : 0/1, key j visible to query i iff j <= i
 *   scale   : multiplies Q K^T (pass 1/sqrt(D) for the usual attention)
 * Supported: D in {64, 128}; any N >= 1; B*H*ceil(N/128) < 2^31.
 */
int tyr_hip_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                           uint64_t B, uint64_t H, uint64_t N, uint64_t D,
                           int causal, float scale, void* stream);

/* Flash-attention forward with grouped queries, sliding window and per-sequence key length.
 *
 * GPU twin of the prefill calls of the reference's models: `lean_torch_sdpa_gqa`
 * (cc/src/tyr.cpp:3913-3949: K / V repeat_interleave'd along the head axis, query head h
 * reads kv head h / (Hq/Hkv); caller Tyr/Model/Qwen/Attention.lean:138),
 * `lean_torch_sdpa_gqa_window` (cc/src/tyr.cpp:3953-4016: key j visible to query i iff
 * j <= i and i - j < window) and `lean_torch_sdpa_gqa_mask` (cc/src/tyr.cpp:4019-4095)
 * for padding masks whose valid keys are a prefix of the sequence.
 *
 *   q, o   : bf16 [B, Hq, N, D]      k, v : bf16 [B, Hkv, N, D], Hq % Hkv == 0
 *   window : 0 = none; > 0 requires causal != 0
 *   kv_lens: device int32 [B] (valid key count of each sequence, clamped to [0, N]) or NULL.
 *            Keys at or beyond it are masked; rows of padded queries are still written
 *            (a row that sees no key at all -- every row of a sequence of length 0 -- gets
 *            O = 0, LSE = -inf; LibTorch returns NaN there).
 * tyr_hip_flash_attn_fwd is this call with Hkv = Hq, window = 0, kv_lens = NULL.
 */
int tyr_hip_flash_attn_fwd_gqa(const void* q, const void* k, const void* v, void* o, float* lse,
                               uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                               int causal, uint64_t window, const int32_t* kv_lens, float scale,
                               void* stream);

/* The forward with an arbitrary per-sequence key mask: `lean_torch_sdpa_gqa_mask`
 * (cc/src/tyr.cpp:4019-4095; mask [batch, seq], 1 = valid key, combined with the causal rule when
 * is_causal) for any mask pattern, e.g. left padding.
 *   key_mask: device uint8 [B, N]; key j of sequence b is visible iff key_mask[b*N + j] != 0.
 * A row that sees no key gets O = 0, LSE = -inf (LibTorch returns NaN there).  Otherwise as
 * tyr_hip_flash_attn_fwd_gqa with window = 0 and no kv_lens.
 */
int tyr_hip_flash_attn_fwd_mask(const void* q, const void* k, const void* v, void* o, float* lse,
                                uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                int causal, const uint8_t* key_mask, float scale, void* stream);

/* ---------------------------------------------------------------------------
 * Flash-attention backward.
 *
 * Replaces the pair `tkMhaH100BwdPrep2Block` + `tkMhaH100Bwd2BlockPartials`
 * (Tyr/GPU/Kernels/MhaH100.lean:197-344; launched from
 * Examples/GPU/RunMhaH100.lean:118-140) for any B, H, N, and the host-side
 * reduction of the per-(kv tile, q tile) partials that runner performs
 * (Examples/GPU/RunMhaH100.lean:131-138): dK and dV come out final.  The
 * values are the gradients autograd returns for
 * `scaled_dot_product_attention` (Examples/GPU/RunMhaH100.lean:56-64).
 *
 *   q, k, v, o, d_o : bf16 [B, H, N, D] row-major contiguous; o and lse are the
 *                     outputs of tyr_hip_flash_attn_fwd for the same q, k, v, causal, scale
 *   lse             : f32 [B, H, N], natural log of the row sums of exp(scaled scores)
 *   dq, dk, dv      : bf16 [B, H, N, D] (written; need not be initialised)
 *   workspace       : device scratch of at least tyr_hip_flash_attn_bwd_workspace_bytes(...)
 *                     bytes, 16-byte aligned; contents need not be initialised
 * Supported: D in {64, 128}; any N >= 1 with N*D*2 < 2^31; B*H*ceil(N/128) < 2^31.
 * The result is deterministic (no atomic accumulation).
 */
size_t tyr_hip_flash_attn_bwd_workspace_bytes(uint64_t B, uint64_t H, uint64_t N, uint64_t D);
int tyr_hip_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o,
                           const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                           uint64_t B, uint64_t H, uint64_t N, uint64_t D,
                           int causal, float scale, void* workspace, size_t workspace_bytes,
                           void* stream);

/* ---------------------------------------------------------------------------
 * GQA decode attention (one query token per sequence), split-KV + LSE combine.
 *
 * GPU twin of `lean_torch_sdpa_gqa_qkv` with q_seq = 1, is_causal = false,
 * enable_gqa = true (cc/src/tyr.cpp:4100-4133; caller
 * Tyr/Model/Qwen/Attention.lean:151-211); query head h reads kv head
 * h / (Hq/Hkv) (repeat_interleave along the head axis).  The packing of the
 * Hq/Hkv query heads of one kv head into one MFMA tile follows
 * Tyr/GPU/Kernels/FlashAttn3.lean:535-624.
 *
 *   q : bf16 [B, Hq, 1, D]
 *   k, v : bf16 [B, Hkv, kv_stride, D]; only rows [0, L) of each (b, kv head) are read.
 *          kv_stride >= L is the allocated cache length (the reference's
 *          [batch, kv_heads, maxLen, head_dim] cache, Tyr/Model/Qwen/Attention.lean:54-68).
 *   o : bf16 [B, Hq, 1, D]      lse : f32 [B, Hq] (may be NULL)
 *   num_splits : KV chunks per (b, kv head); 0 = choose automatically.
 *   workspace  : device scratch of at least tyr_hip_gqa_decode_workspace_bytes(...) bytes,
 *                16-byte aligned; contents need not be initialised.
 * Supported: D in {64, 128}; 1 <= Hq/Hkv <= 16 with Hq % Hkv == 0; L >= 1; num_splits <= 64.
 */
size_t tyr_hip_gqa_decode_workspace_bytes(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L,
                                          uint64_t D, uint64_t num_splits);
/* The split count the library uses when num_splits == 0 is passed. */
uint64_t tyr_hip_gqa_decode_auto_splits(uint64_t B, uint64_t Hkv, uint64_t L);
int tyr_hip_gqa_decode(const void* q, const void* k, const void* v, void* o, float* lse,
                       uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                       uint64_t kv_stride, float scale, uint64_t num_splits,
                       void* workspace, size_t workspace_bytes, void* stream);

/* tyr_hip_gqa_decode without a workspace argument and without any allocation.
 *
 * No counterpart in the reference.  It is for callers that cannot allocate device memory around
 * the call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The partial results of the split pass go to a fixed device array of
 * TYR_HIP_GQA_DECODE_STATIC_SCRATCH_BYTES bytes that the library holds on every GPU it runs on
 * until the process ends; the call makes no hipMalloc / hipFree and uses no allocating library
 * routine.  Arguments and results are those of tyr_hip_gqa_decode (same kernels).
 *
 * Limit: tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, L, D, num_splits) must not exceed
 * TYR_HIP_GQA_DECODE_STATIC_SCRATCH_BYTES, else TYR_HIP_ERR_WORKSPACE is returned and nothing is
 * launched (B * Hq * num_splits <= 16131 at D = 128).
 * Every call on one GPU uses the same array: calls that overlap in time on one GPU (different
 * streams, different threads) race on it; calls on one stream are ordered and safe.  Nothing in
 * the array has to start at zero (the split pass writes every partial the combine pass reads).
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make that call
 * outside stream capture.
 */
#define TYR_HIP_GQA_DECODE_STATIC_SCRATCH_BYTES ((size_t)8 << 20)
int tyr_hip_gqa_decode_static(const void* q, const void* k, const void* v, void* o, float* lse,
                              uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                              uint64_t kv_stride, float scale, uint64_t num_splits, void* stream);

/* Flash-attention backward for the forward of tyr_hip_flash_attn_fwd_gqa (same q, k, v, causal,
 * window, kv_lens, scale; o and lse its outputs).  dq : bf16 [B, Hq, N, D]; dk, dv : bf16
 * [B, Hkv, N, D], each summed over the Hq/Hkv query heads that read that kv head (the gradient of
 * the reference's repeat_interleave, cc/src/tyr.cpp:3930-3936).  Rows of dk / dv at or beyond a
 * sequence's length are written as zero.  workspace: tyr_hip_flash_attn_bwd_workspace_bytes(B, Hq, N, D).
 * Supported additionally: (Hq/Hkv) * N * D * 2 < 2^31.  tyr_hip_flash_attn_bwd is this call with
 * Hkv = Hq, window = 0, kv_lens = NULL.
 */
int tyr_hip_flash_attn_bwd_gqa(const void* q, const void* k, const void* v, const void* o,
                               const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                               uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                               int causal, uint64_t window, const int32_t* kv_lens, float scale,
                               void* workspace, size_t workspace_bytes, void* stream);

/* Backward of tyr_hip_flash_attn_fwd_mask (autograd of `lean_torch_sdpa_gqa_mask`,
 * cc/src/tyr.cpp:4019-4095): hidden keys receive dk = dv = 0, rows that saw no key dq = 0. */
int tyr_hip_flash_attn_bwd_mask(const void* q, const void* k, const void* v, const void* o,
                                const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                                uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                int causal, const uint8_t* key_mask, float scale,
                                void* workspace, size_t workspace_bytes, void* stream);

/* GQA decode with a per-sequence cache length and / or a sliding window.
 *
 * Decode-time (one query token) form of `lean_torch_sdpa_gqa_mask` (padding mask: the valid
 * keys of sequence b are a prefix of the cache; cc/src/tyr.cpp:4019-4095) and of
 * `lean_torch_sdpa_gqa_window` (position i attends to j <= i with i - j < window;
 * cc/src/tyr.cpp:3953-4016), the query standing at the last valid position:
 * sequence b attends to cache rows [max(0, len_b - window), len_b), len_b = kv_lens[b].
 *
 *   kv_lens : device int32 [B], each clamped to [0, L]; NULL = every sequence has L rows.
 *             A sequence of length 0 gets O = 0 and LSE = -inf.
 *   window  : 0 = unbounded
 *   L       : upper bound of the lengths (sizes the splits and the workspace)
 * Everything else as tyr_hip_gqa_decode, which is this call with kv_lens = NULL, window = 0.
 */
int tyr_hip_gqa_decode_varlen(const void* q, const void* k, const void* v, void* o, float* lse,
                              uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                              uint64_t kv_stride, const int32_t* kv_lens, uint64_t window,
                              float scale, uint64_t num_splits, void* workspace,
                              size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Decode step: rotary embedding of the new q and k, append of k and v to the cache.
 *
 * Fuses what `QwenAttention.forwardStep` does between the projections and the
 * attention call (Tyr/Model/Qwen/Attention.lean:172-196): `rotary.applyRotaryEmb`
 * on the single-token q and k (cc/src/tyr.cpp:3837-3873) and `data.sliceScatter`
 * of k and v into row `pos` of the preallocated cache.  tyr_hip_gqa_decode with
 * L = pos + 1 and the same kv_stride then reads the cache in place.
 *
 *   q          : bf16 [B, Hq, D]   (the [B,1,Hq,D] projection output; same bytes as [B,Hq,1,D])
 *   k_new,v_new: bf16 [B, Hkv, D]
 *   cos, sin   : f32 [D/2], the row of the rotary table for position `pos`
 *   q_out      : bf16 [B, Hq, D] (rotated q; may alias q)
 *   k_cache, v_cache : bf16 [B, Hkv, kv_stride, D]; row `pos` of every (b, kv head) is written
 * Supported: D % 16 == 0; pos < kv_stride.
 */
int tyr_hip_decode_rope_append(const void* q, const void* k_new, const void* v_new,
                               const float* cos, const float* sin, void* q_out,
                               void* k_cache, void* v_cache,
                               uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t D,
                               uint64_t kv_stride, uint64_t pos, void* stream);

/* ---------------------------------------------------------------------------
 * Rotary embedding (prefill form).
 *
 * GPU twin of `lean_torch_apply_rotary_emb` (cc/src/tyr.cpp:3837-3873; Lean decl
 * Tyr/Torch.lean:1044) and replacement of the DSL kernel `rotaryFwd`
 * (Tyr/GPU/Kernels/Rotary.lean:13-66, one f32 64x64 tile) for any shape:
 * x = [x1 | x2] split in halves along D; y1 = x1 cos - x2 sin; y2 = x1 sin + x2 cos.
 *
 *   x, y     : [B, S, H, D], f32 (dtype = TYR_HIP_F32) or bf16 (TYR_HIP_BF16); y may alias x
 *   cos, sin : f32 [S, D/2]
 * Supported: D % 8 == 0 (f32) / D % 16 == 0 (bf16).
 */
enum tyr_hip_dtype { TYR_HIP_F32 = 0, TYR_HIP_BF16 = 1 };
int tyr_hip_rope_fwd(const void* x, const float* cos, const float* sin, void* y,
                     uint64_t B, uint64_t S, uint64_t H, uint64_t D, int dtype, void* stream);

/* ---------------------------------------------------------------------------
 * Fused residual add + LayerNorm.
 *
 * Replaces the DSL kernel `tkFusedLayerNormResidual1024`
 * (Tyr/GPU/Kernels/FusedLayerNorm.lean:28-140; runner Examples/GPU/RunLayerNorm.lean:60-75)
 * for any row count and any d_model % 8 == 0 up to 8192:
 *   out_resid = bf16(x + residual)
 *   out       = bf16((out_resid - mean) * rsqrt(var + eps) * weight + bias)
 * with mean / var over the whole row of the rounded out_resid, in f32.
 *
 *   x, residual, out, out_resid : bf16 [rows, d_model]      weight, bias : bf16 [d_model]
 */
int tyr_hip_layernorm_residual(const void* x, const void* residual, const void* weight,
                               const void* bias, void* out, void* out_resid,
                               uint64_t rows, uint64_t d_model, float eps, void* stream);

/* ---------------------------------------------------------------------------
 * Device-to-device copy kernel.
 *
 * Replaces the DSL kernel `copy64x64` (Tyr/GPU/Kernels/Copy.lean:16-27; runner
 * Examples/GPU/RunCopy.lean) for any byte count.  src and dst must be 16-byte
 * aligned and must not overlap.
 */
int tyr_hip_copy(const void* src, void* dst, size_t bytes, void* stream);

/* ---------------------------------------------------------------------------
 * bf16 GEMM, f32 accumulation, bf16 output:  C = A B  (trans_b = 0, B is [K, N])
 *                                            C = A B^T (trans_b = 1, B is [N, K]).
 *
 * Replaces `tkH100Bf16GemmFwd` (Tyr/GPU/Kernels/Bf16Gemm.lean:64-73) over
 * `tiledAccumulator` (Tyr/GPU/Kernels/GemmCommon.lean:22-69, the N x K form)
 * and `simpleGemm` (Tyr/GPU/Kernels/Examples.lean:23-65, the K x N form);
 * GPU twin of `lean_torch_mm` (cc/src/tyr.cpp:1602-1607).
 *
 *   a : bf16 [M, K]   b : bf16 [K, N] or [N, K]   c : bf16 [M, N]
 * Supported: M, N, K >= 1 with K % 8 == 0 and N % 8 == 0 (16-byte rows).
 */
int tyr_hip_gemm_bf16(const void* a, const void* b, void* c,
                      uint64_t M, uint64_t N, uint64_t K, int trans_b, void* stream);

/* Batched form: `batch` independent products C_i = A_i B_i in one launch, entry i at
 * a + i*stride_a, b + i*stride_b, c + i*stride_c (strides in elements, multiples of 8).
 * GPU twin of `lean_torch_matmul` (cc/src/tyr.cpp:1565-1570) for operands of rank > 2:
 * [batch, M, K] x [batch, K, N] with stride_a = M*K, stride_b = K*N, stride_c = M*N, and the
 * broadcast case [batch, M, K] x [K, N] with stride_b = 0.  batch <= 65535; stride_c >= M*N.
 * tyr_hip_gemm_bf16 is this call with batch = 1.
 */
int tyr_hip_gemm_bf16_batched(const void* a, const void* b, void* c, uint64_t batch,
                              uint64_t M, uint64_t N, uint64_t K,
                              uint64_t stride_a, uint64_t stride_b, uint64_t stride_c,
                              int trans_b, void* stream);

/* Test switch (no counterpart in the reference).  The bf16 and fp8 GEMMs have a fast kernel and a
 * general (register-staged) kernel that otherwise serves only shapes whose 256-row panels or whose
 * [K, N] B exceed 32-bit byte offsets.  on != 0 sends every shape through the general kernels,
 * process-wide, until switched off again; the previous setting is returned.  The initial setting is
 * "on" iff the environment variable TYR_HIP_GEMM_GENERAL exists when the first GEMM is launched. */
int tyr_hip_gemm_force_general(int on);

/* Launch-shape switch of the forward attention kernels (no counterpart in the reference).  A forward launch
 * starts either one workgroup per (head, query-tile job), or -- on != 0 -- two persistent workgroups per CU
 * that walk the jobs.  Results are bit-identical; only the timing differs (which of the two is faster depends on
 * the shape and, by a few per cent, on the individual device).  Process-wide until changed again; the previous
 * setting is returned.  The initial setting is "on" iff the environment variable TYR_HIP_FA_PERSISTENT is "1"
 * when the first forward is launched. */
int tyr_hip_flash_attn_fwd_persistent(int on);

/* ---------------------------------------------------------------------------
 * FP8 E4M3 GEMM with per-tensor f32 scales, bf16 output:
 *     C = bf16( scale_a * scale_b * (Aq Bq) ),  f32 accumulation, scale in the epilogue.
 *
 * Replaces `gemmFp8E4M3Fwd` / `tkH100Fp8ScaledGemmFwd`
 * (Tyr/GPU/Kernels/PrecisionGemm.lean:97-115,178-189) with the scalar epilogue of
 * `applyGlobalScalar` (Tyr/GPU/Kernels/GemmCommon.lean:135-144).
 *
 *   aq : e4m3 [M, K]   bq : e4m3 [K, N] (trans_b = 0) or [N, K] (trans_b = 1)   c : bf16 [M, N]
 * Supported: M, N, K >= 1 with K % 16 == 0 and N % 16 == 0 (16-byte rows).
 */
int tyr_hip_gemm_fp8(const void* aq, const void* bq, void* c,
                     uint64_t M, uint64_t N, uint64_t K,
                     float scale_a, float scale_b, int trans_b, void* stream);

/* The other epilogues of the reference's fp8 GEMM family on the same mainloop:
 *     C[m, n] = out_dtype( scale * row_scale[m] * col_scale[n] * sum_k Aq[m, k] Bq[k, n] )
 *   - `tkH100Fp8E4M3GemmFwd` (Tyr/GPU/Kernels/PrecisionGemm.lean:78-89): E4M3 output, no scales
 *     (out_dtype = TYR_HIP_OUT_E4M3; round to nearest even, saturating at +-448);
 *   - `tkH100Fp8ScaledGemmFwd` (Tyr/GPU/Kernels/PrecisionGemm.lean:97-115 with the epilogue of
 *     Tyr/GPU/Kernels/GemmCommon.lean:83-133): per-row and per-column f32 dequantisation scales, f32 output
 *     (out_dtype = TYR_HIP_OUT_F32, row_scale [M], col_scale [N]);
 *   - tyr_hip_gemm_fp8 is this call with scale = scale_a * scale_b, no vectors, TYR_HIP_OUT_BF16.
 * row_scale / col_scale: device f32 vectors or NULL (= all ones); col_scale 16-byte aligned.
 * c: [M, N] of the output type.  Shapes as tyr_hip_gemm_fp8.
 */
enum tyr_hip_out_dtype { TYR_HIP_OUT_BF16 = 0, TYR_HIP_OUT_F32 = 1, TYR_HIP_OUT_E4M3 = 2 };
int tyr_hip_gemm_fp8_ex(const void* aq, const void* bq, void* c,
                        uint64_t M, uint64_t N, uint64_t K,
                        float scale, const float* row_scale, const float* col_scale, int out_dtype,
                        int trans_b, void* stream);

/* ---------------------------------------------------------------------------
 * The element-wise half of the attention train step, fused.
 *
 * The reference's `oneKernelTrainStep` (Examples/GPU/RunMhaH100Train.lean:77-93) surrounds its forward
 * and backward kernels with LibTorch element-wise calls; these two entry points are those chains as one
 * streaming pass each, with bit-identical results for dO and the parameters.
 *
 * tyr_hip_mse_loss_grad -- `lossAndGradOut` (:60-67):
 *     diff = f32(out) - f32(target);  *loss = 0.5 * mean(diff^2);  d_out = bf16(diff / n)
 *   out, target, d_out : bf16 [n] (any shape, n elements, n % 8 == 0);  loss : device f32 scalar
 *   workspace : tyr_hip_mse_loss_grad_workspace_bytes(n) bytes of device scratch (per-workgroup partial sums)
 * tyr_hip_sgd_step -- `sgdUpdate` (:69-70) plus the bf16 cast of the next step (:83-85):
 *     param_out = param - (f32(grad) * lr);  param_out_bf16 = bf16(param_out)  (skipped when NULL)
 *   param, param_out : f32 [n] (param_out may alias param);  grad, param_out_bf16 : bf16 [n];  n % 8 == 0
 */
size_t tyr_hip_mse_loss_grad_workspace_bytes(uint64_t n);
int tyr_hip_mse_loss_grad(const void* out, const void* target, void* d_out, float* loss, uint64_t n,
                          void* workspace, size_t workspace_bytes, void* stream);
int tyr_hip_sgd_step(const float* param, const void* grad, float lr, float* param_out, void* param_out_bf16,
                     uint64_t n, void* stream);

/* ---------------------------------------------------------------------------
 * Calibration: the MFMA rate this device sustains on the caller's operand bits.
 *
 * No counterpart in the reference; it belongs to the measurement side, where the reference's
 * runners print a torch figure beside the kernel's (Examples/GPU/RunMhaH100Train.lean:217-288).
 * Every wave of `workgroups` 4-wave workgroups loads 8 operand fragments from `operands` once and
 * then issues only MFMAs (32x32x16 bf16 or 32x32x64 E4M3), `iters` rounds of 16.  *flop_per_launch
 * receives the floating-point operations of one launch.  `sink` (device memory of `sink_bytes` bytes) takes 256
 * floats per workgroup; a smaller buffer is refused with TYR_HIP_ERR_WORKSPACE before anything is launched.
 */
enum tyr_hip_mfma_type { TYR_HIP_MFMA_BF16 = 0, TYR_HIP_MFMA_E4M3 = 1 };
int tyr_hip_mfma_sustain(const void* operands, size_t operand_bytes, int dtype, uint64_t workgroups,
                         uint64_t iters, float* sink, size_t sink_bytes, double* flop_per_launch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TYR_HIP_H */
