/*
 * tyr_oracle.c -- CPU restatement of the arithmetic of Tyr's GPU kernel hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against; it is never linked into, imported by, or called from the
 * shipped library or its host-side mirror.  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load it.
 *
 * Every function restates, in plain scalar C, one algorithm of the reference
 * (paths are relative to the reference checkout):
 *
 *   oracle_attn_fwd_tiled   Tyr/GPU/Kernels/MhaH100.lean:71-128 (kernel body),
 *                           Tyr/GPU/Codegen/Macros.lean:121-163 (onlineSoftmax,
 *                           finalizeSoftmax, computeLSE), causal semantics of
 *                           cc/src/tyr.cpp:2563-2589 (is_causal=true).
 *   oracle_attn_fwd_f64     textbook softmax(QK^T*scale + mask) V in double; the
 *                           same math as Examples/GPU/RunFlashAttn.lean:31-48
 *                           (reference values for O and LSE).
 *   oracle_attn_fwd_f64_ex  the same with the grouped-query head mapping of
 *                           cc/src/tyr.cpp:3913-3949, the window rule of :3953-4016 and a
 *                           prefix padding mask (:4019-4095).
 *   oracle_attn_bwd_f64     Tyr/GPU/Kernels/MhaH100.lean:197-344 (backward prep
 *                           d = rowsum(dO o O) and the dQ / dK / dV products:
 *                           P = exp(S*scale - lse), dP = dO V^T, dS = P o (dP - d),
 *                           dV = P^T dO, dK = scale dS^T Q, dQ = scale dS K), in
 *                           double; reference values as Examples/GPU/RunMhaH100.lean:56-64
 *                           takes them from autograd.
 *   oracle_attn_*_f64_mask  the _ex functions with an arbitrary per-sequence key mask as well
 *                           (cc/src/tyr.cpp:4019-4095: mask [batch, seq], 1 = valid key).
 *   oracle_attn_bwd_f64_ex  the same with grouped queries (dK / dV summed over the query
 *                           heads of a kv head: the gradient of repeat_interleave), window
 *                           and prefix key lengths.
 *   oracle_gqa_decode       cc/src/tyr.cpp:4100-4133 (repeat_interleave mapping),
 *                           Tyr/GPU/Kernels/FlashAttn3.lean:535-624 (q-head packing),
 *                           split/merge algebra of Tyr/GPU/Kernels/RingAttn.lean
 *                           (online-softmax merge of partial (O, m, l)).
 *   oracle_gemm_bf16        Tyr/GPU/Kernels/GemmCommon.lean:22-69 (f32 accumulate,
 *                           bf16 epilogue), Tyr/GPU/Kernels/Examples.lean:23-65 (NN),
 *                           cc/src/tyr.cpp:1602-1607 (torch::mm).
 *   oracle_gemm_fp8         Tyr/GPU/Kernels/PrecisionGemm.lean:97-115,178-189 and
 *                           Tyr/GPU/Kernels/GemmCommon.lean:135-144 (scalar scale in
 *                           the f32 epilogue, bf16 out).
 *   oracle_rope             cc/src/tyr.cpp:3837-3873 (lean_torch_apply_rotary_emb: halves
 *                           split, y1 = x1 cos - x2 sin, y2 = x1 sin + x2 cos, f32
 *                           arithmetic, result in x's dtype); Tyr/GPU/Kernels/Rotary.lean:13-66.
 *   oracle_layernorm_residual  Tyr/GPU/Kernels/FusedLayerNorm.lean:28-140 (out_resid =
 *                           bf16(x + residual); row statistics of the rounded sum;
 *                           normalise, weight, bias; bf16 out), in double.
 *   oracle_e4m3_*           OCP FP8 E4M3 ("e4m3fn": bias 7, max 448, no inf, NaN at
 *                           S.1111.111); dtype tag at Tyr/GPU/Types.lean:21-58.
 *
 * Pinning status (see tests/test_oracle_*.py): every function here is checked
 * against an independent statement of the same math -- float64 brute force on
 * small inputs, the LibTorch routines the reference calls
 * (scaled_dot_product_attention, mm, logsumexp, float8_e4m3fn casts), closed
 * forms (identity / permutation operands, one-hot attention, the 256-entry
 * E4M3 table) and invariants (tile-size and split-count independence, causal
 * future-independence, decode == last row of causal prefill).  The reference
 * holds no committed golden vectors for this path, so none are used.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

/* ---------------------------------------------------------------- bf16 -- */

static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even, NaN kept quiet; same rule as torch's .to(bfloat16) */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

static inline float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
float oracle_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* ---------------------------------------------------------------- e4m3 -- */

/* OCP E4M3 decode: sign(1) exp(4, bias 7) mant(3); exp=0 subnormal (2^-6 * m/8);
 * exp=15,mant=7 is NaN; there is no infinity; largest finite = 1.75 * 2^8 = 448. */
float oracle_e4m3_decode(uint8_t c) {
    int s = c >> 7, e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 15 && m == 7) return NAN;
    if (e == 0) v = ldexpf((float)m, -9);
    else        v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return s ? -v : v;
}

/* Saturating round-to-nearest-even encode (finite inputs clamp to +-448). */
uint8_t oracle_e4m3_encode(float f) {
    if (isnan(f)) return 0x7f;
    uint8_t s = signbit(f) ? 0x80 : 0;
    float a = fabsf(f);
    if (a >= 448.0f) return (uint8_t)(s | 0x7e);
    if (a < ldexpf(1.0f, -10)) return s;  /* below half the smallest subnormal (ties-to-even -> 0) */
    int e;
    (void)frexpf(a, &e);          /* a = fr * 2^e, fr in [0.5,1) -> unbiased exponent e-1 */
    int ue = e - 1;
    if (ue < -6) ue = -6;         /* subnormal range shares the exponent of 2^-6 */
    float q = ldexpf(a, 3 - ue);  /* a in units of the local ulp = 2^(ue-3) */
    float r = nearbyintf(q);      /* default rounding mode: to nearest, ties to even */
    int mant = (int)r;            /* 8..16 for normals, 0..8 for subnormals */
    int be = ue + 7;
    if (ue == -6 && mant < 8) be = 0;           /* stays subnormal */
    else { if (mant == 16) { mant = 8; be += 1; } mant -= 8; }
    if (be >= 16 || (be == 15 && mant == 7)) return (uint8_t)(s | 0x7e);
    return (uint8_t)(s | (be << 3) | mant);
}

/* ---------------------------------------------------- attention forward -- */

/* Textbook attention in double precision.  q,k,v: bf16 bit patterns,
 * [B,H,N,D] contiguous; o: f32 [B,H,N,D]; lse: f32 [B,H,N] = ln sum_j exp(s_ij). */
void oracle_attn_fwd_f64(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                         float* o, float* lse,
                         int64_t B, int64_t H, int64_t N, int64_t D,
                         int causal, double scale) {
    #pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t bh = 0; bh < B * H; ++bh) {
        for (int64_t i = 0; i < N; ++i) {
            const uint16_t* qr = q + (bh * N + i) * D;
            int64_t jmax = causal ? i + 1 : N;
            double* s = (double*)malloc(sizeof(double) * (size_t)jmax);
            double m = -INFINITY;
            for (int64_t j = 0; j < jmax; ++j) {
                const uint16_t* kr = k + (bh * N + j) * D;
                double acc = 0.0;
                for (int64_t d = 0; d < D; ++d) acc += (double)bf16_to_f32(qr[d]) * (double)bf16_to_f32(kr[d]);
                s[j] = acc * scale;
                if (s[j] > m) m = s[j];
            }
            double l = 0.0;
            for (int64_t j = 0; j < jmax; ++j) { s[j] = exp(s[j] - m); l += s[j]; }
            for (int64_t d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int64_t j = 0; j < jmax; ++j) acc += s[j] * (double)bf16_to_f32(v[(bh * N + j) * D + d]);
                o[(bh * N + i) * D + d] = (float)(acc / l);
            }
            if (lse) lse[bh * N + i] = (float)(log(l) + m);
            free(s);
        }
    }
}

/* Textbook attention in double precision with grouped queries, a sliding window and a
 * per-sequence key length: q [B,Hq,N,D]; k, v [B,Hkv,N,D]; query head h reads kv head
 * h / (Hq/Hkv) (repeat_interleave along the head axis, cc/src/tyr.cpp:3930-3936); key j is
 * visible to query i iff j < kv_lens[b] (if given), j <= i (if causal) and i - j < window
 * (if window > 0; cc/src/tyr.cpp:3980-3996).  A row without any visible key gets O = 0,
 * LSE = -inf. */
/* key_mask: uint8 [B,N], nonzero = key may be attended to (the padding mask of
 * cc/src/tyr.cpp:4019-4095, any pattern), or NULL.  A row whose every key is hidden gives
 * O = 0, LSE = -inf (LibTorch returns NaN there). */
void oracle_attn_fwd_f64_mask(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                              float* o, float* lse, int64_t B, int64_t Hq, int64_t Hkv, int64_t N,
                              int64_t D, int causal, int64_t window, const int32_t* kv_lens,
                              const uint8_t* key_mask, double scale) {
    const int64_t G = Hq / Hkv;
    #pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t bh = 0; bh < B * Hq; ++bh) {
        for (int64_t i = 0; i < N; ++i) {
            const int64_t b = bh / Hq, h = bh % Hq, kvh = b * Hkv + h / G;
            const uint16_t* qr = q + (bh * N + i) * D;
            int64_t len = kv_lens ? kv_lens[b] : N;
            if (len > N) len = N;
            if (len < 0) len = 0;                      /* an empty sequence: O = 0, LSE = -inf, no gradients */
            int64_t jhi = causal ? (i + 1 < len ? i + 1 : len) : len;       /* exclusive */
            int64_t jlo = window > 0 ? (i - window + 1 > 0 ? i - window + 1 : 0) : 0;
            float* orow = o + (bh * N + i) * D;
            if (jlo >= jhi) {
                for (int64_t d = 0; d < D; ++d) orow[d] = 0.0f;
                if (lse) lse[bh * N + i] = -INFINITY;
                continue;
            }
            double* s = (double*)malloc(sizeof(double) * (size_t)(jhi - jlo));
            double m = -INFINITY;
            for (int64_t j = jlo; j < jhi; ++j) {
                const uint16_t* kr = k + (kvh * N + j) * D;
                double acc = 0.0;
                for (int64_t d = 0; d < D; ++d) acc += (double)bf16_to_f32(qr[d]) * (double)bf16_to_f32(kr[d]);
                s[j - jlo] = (key_mask && !key_mask[b * N + j]) ? -INFINITY : acc * scale;
                if (s[j - jlo] > m) m = s[j - jlo];
            }
            if (m == -INFINITY) {                      /* every key in range is hidden */
                for (int64_t d = 0; d < D; ++d) orow[d] = 0.0f;
                if (lse) lse[bh * N + i] = -INFINITY;
                free(s);
                continue;
            }
            double l = 0.0;
            for (int64_t j = jlo; j < jhi; ++j) { s[j - jlo] = exp(s[j - jlo] - m); l += s[j - jlo]; }
            for (int64_t d = 0; d < D; ++d) {
                double acc = 0.0;
                for (int64_t j = jlo; j < jhi; ++j) acc += s[j - jlo] * (double)bf16_to_f32(v[(kvh * N + j) * D + d]);
                orow[d] = (float)(acc / l);
            }
            if (lse) lse[bh * N + i] = (float)(log(l) + m);
            free(s);
        }
    }
}

void oracle_attn_fwd_f64_ex(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                            float* o, float* lse, int64_t B, int64_t Hq, int64_t Hkv, int64_t N,
                            int64_t D, int causal, int64_t window, const int32_t* kv_lens, double scale) {
    oracle_attn_fwd_f64_mask(q, k, v, o, lse, B, Hq, Hkv, N, D, causal, window, kv_lens, NULL, scale);
}

/* Attention backward in double precision.  q,k,v,d_o: bf16 bit patterns [B,H,N,D];
 * dq,dk,dv: f32 [B,H,N,D].  The forward quantities (P, O) are recomputed here in double,
 * so the result is the exact gradient of oracle_attn_fwd_f64's O contracted with d_o. */
void oracle_attn_bwd_f64(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                         const uint16_t* d_o, float* dq, float* dk, float* dv,
                         int64_t B, int64_t H, int64_t N, int64_t D,
                         int causal, double scale) {
    #pragma omp parallel for schedule(dynamic)
    for (int64_t bh = 0; bh < B * H; ++bh) {
        const uint16_t* qh = q + bh * N * D;
        const uint16_t* kh = k + bh * N * D;
        const uint16_t* vh = v + bh * N * D;
        const uint16_t* gh = d_o + bh * N * D;
        double* dka = (double*)calloc((size_t)(N * D), sizeof(double));
        double* dva = (double*)calloc((size_t)(N * D), sizeof(double));
        double* p = (double*)malloc(sizeof(double) * (size_t)N);
        double* dp = (double*)malloc(sizeof(double) * (size_t)N);
        double* dqa = (double*)malloc(sizeof(double) * (size_t)D);
        for (int64_t i = 0; i < N; ++i) {
            const int64_t jmax = causal ? i + 1 : N;
            double m = -INFINITY;
            for (int64_t j = 0; j < jmax; ++j) {
                double acc = 0.0;
                for (int64_t d = 0; d < D; ++d)
                    acc += (double)bf16_to_f32(qh[i * D + d]) * (double)bf16_to_f32(kh[j * D + d]);
                p[j] = acc * scale;
                if (p[j] > m) m = p[j];
            }
            double l = 0.0;
            for (int64_t j = 0; j < jmax; ++j) { p[j] = exp(p[j] - m); l += p[j]; }
            for (int64_t j = 0; j < jmax; ++j) p[j] /= l;
            /* dP_j = dO_i . V_j ; delta = sum_j P_j dP_j  (= dO_i . O_i) */
            double delta = 0.0;
            for (int64_t j = 0; j < jmax; ++j) {
                double acc = 0.0;
                for (int64_t d = 0; d < D; ++d)
                    acc += (double)bf16_to_f32(gh[i * D + d]) * (double)bf16_to_f32(vh[j * D + d]);
                dp[j] = acc;
                delta += p[j] * acc;
            }
            for (int64_t d = 0; d < D; ++d) dqa[d] = 0.0;
            for (int64_t j = 0; j < jmax; ++j) {
                const double ds = p[j] * (dp[j] - delta) * scale;
                for (int64_t d = 0; d < D; ++d) {
                    dqa[d] += ds * (double)bf16_to_f32(kh[j * D + d]);
                    dka[j * D + d] += ds * (double)bf16_to_f32(qh[i * D + d]);
                    dva[j * D + d] += p[j] * (double)bf16_to_f32(gh[i * D + d]);
                }
            }
            for (int64_t d = 0; d < D; ++d) dq[(bh * N + i) * D + d] = (float)dqa[d];
        }
        for (int64_t x = 0; x < N * D; ++x) {
            dk[bh * N * D + x] = (float)dka[x];
            dv[bh * N * D + x] = (float)dva[x];
        }
        free(dka); free(dva); free(p); free(dp); free(dqa);
    }
}

/* Attention backward in double precision with grouped queries, sliding window and per-sequence
 * key length (visibility rule of oracle_attn_fwd_f64_ex).  dq: f32 [B,Hq,N,D]; dk, dv: f32
 * [B,Hkv,N,D], each the sum over the Hq/Hkv query heads that read that kv head (the gradient of
 * repeat_interleave is that sum).  Rows without a visible key contribute nothing. */
void oracle_attn_bwd_f64_mask(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                              const uint16_t* d_o, float* dq, float* dk, float* dv,
                              int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                              int causal, int64_t window, const int32_t* kv_lens,
                              const uint8_t* key_mask, double scale) {
    const int64_t G = Hq / Hkv;
    #pragma omp parallel for schedule(dynamic)
    for (int64_t bk = 0; bk < B * Hkv; ++bk) {
        const int64_t b = bk / Hkv, kvh = bk % Hkv;
        const uint16_t* kh = k + bk * N * D;
        const uint16_t* vh = v + bk * N * D;
        int64_t len = kv_lens ? kv_lens[b] : N;
        if (len > N) len = N;
        if (len < 0) len = 0;                      /* an empty sequence: O = 0, LSE = -inf, no gradients */
        double* dka = (double*)calloc((size_t)(N * D), sizeof(double));
        double* dva = (double*)calloc((size_t)(N * D), sizeof(double));
        double* p = (double*)malloc(sizeof(double) * (size_t)N);
        double* dp = (double*)malloc(sizeof(double) * (size_t)N);
        double* dqa = (double*)malloc(sizeof(double) * (size_t)D);
        for (int64_t hq = 0; hq < G; ++hq) {
            const int64_t bh = b * Hq + kvh * G + hq;
            const uint16_t* qh = q + bh * N * D;
            const uint16_t* gh = d_o + bh * N * D;
            for (int64_t i = 0; i < N; ++i) {
                const int64_t jhi = causal ? (i + 1 < len ? i + 1 : len) : len;
                const int64_t jlo = window > 0 ? (i - window + 1 > 0 ? i - window + 1 : 0) : 0;
                for (int64_t d = 0; d < D; ++d) dqa[d] = 0.0;
                if (jlo < jhi) {
                    double m = -INFINITY;
                    for (int64_t j = jlo; j < jhi; ++j) {
                        double acc = 0.0;
                        for (int64_t d = 0; d < D; ++d)
                            acc += (double)bf16_to_f32(qh[i * D + d]) * (double)bf16_to_f32(kh[j * D + d]);
                        p[j] = (key_mask && !key_mask[b * N + j]) ? -INFINITY : acc * scale;
                        if (p[j] > m) m = p[j];
                    }
                    if (m == -INFINITY) {              /* every key hidden: the row contributes nothing */
                        for (int64_t d = 0; d < D; ++d) dq[(bh * N + i) * D + d] = 0.0f;
                        continue;
                    }
                    double l = 0.0;
                    for (int64_t j = jlo; j < jhi; ++j) { p[j] = exp(p[j] - m); l += p[j]; }
                    double delta = 0.0;
                    for (int64_t j = jlo; j < jhi; ++j) {
                        p[j] /= l;
                        double acc = 0.0;
                        for (int64_t d = 0; d < D; ++d)
                            acc += (double)bf16_to_f32(gh[i * D + d]) * (double)bf16_to_f32(vh[j * D + d]);
                        dp[j] = acc;
                        delta += p[j] * acc;
                    }
                    for (int64_t j = jlo; j < jhi; ++j) {
                        const double ds = p[j] * (dp[j] - delta) * scale;
                        for (int64_t d = 0; d < D; ++d) {
                            dqa[d] += ds * (double)bf16_to_f32(kh[j * D + d]);
                            dka[j * D + d] += ds * (double)bf16_to_f32(qh[i * D + d]);
                            dva[j * D + d] += p[j] * (double)bf16_to_f32(gh[i * D + d]);
                        }
                    }
                }
                for (int64_t d = 0; d < D; ++d) dq[(bh * N + i) * D + d] = (float)dqa[d];
            }
        }
        for (int64_t x = 0; x < N * D; ++x) {
            dk[bk * N * D + x] = (float)dka[x];
            dv[bk * N * D + x] = (float)dva[x];
        }
        free(dka); free(dva); free(p); free(dp); free(dqa);
    }
}

void oracle_attn_bwd_f64_ex(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                            const uint16_t* d_o, float* dq, float* dk, float* dv,
                            int64_t B, int64_t Hq, int64_t Hkv, int64_t N, int64_t D,
                            int causal, int64_t window, const int32_t* kv_lens, double scale) {
    oracle_attn_bwd_f64_mask(q, k, v, d_o, dq, dk, dv, B, Hq, Hkv, N, D, causal, window, kv_lens, NULL, scale);
}

/* Tiled online-softmax attention in the reference kernel's order of operations:
 *   S = Q K_j^T (f32 acc of bf16 products) ; S *= scale ; mask ;
 *   m' = max(m,rowmax S) ; alpha = exp(m-m') ; O *= alpha ; l *= alpha ;
 *   P = exp(S-m') ; l += rowsum(P) ; O += bf16(P) V_j ; finally O /= l,
 *   LSE = ln l + m, O rounded to bf16.
 * o_bf16: bf16 bit patterns [B,H,N,D]; lse f32 [B,H,N]; tile_kv = KV tile rows. */
void oracle_attn_fwd_tiled(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                           uint16_t* o_bf16, float* lse,
                           int64_t B, int64_t H, int64_t N, int64_t D,
                           int causal, float scale, int64_t tile_kv) {
    if (tile_kv <= 0) tile_kv = 64;
    #pragma omp parallel for schedule(dynamic)
    for (int64_t row = 0; row < B * H * N; ++row) {
        int64_t bh = row / N, i = row % N;
        const uint16_t* qr = q + row * D;
        float* acc = (float*)calloc((size_t)D, sizeof(float));
        float* s = (float*)malloc(sizeof(float) * (size_t)tile_kv);
        float m = -INFINITY, l = 0.0f;
        int64_t kv_end = causal ? i + 1 : N;
        for (int64_t j0 = 0; j0 < kv_end; j0 += tile_kv) {
            int64_t jn = j0 + tile_kv < N ? tile_kv : N - j0;
            float tmax = -INFINITY;
            for (int64_t jj = 0; jj < jn; ++jj) {
                int64_t j = j0 + jj;
                const uint16_t* kr = k + (bh * N + j) * D;
                float a = 0.0f;
                for (int64_t d = 0; d < D; ++d) a += bf16_to_f32(qr[d]) * bf16_to_f32(kr[d]);
                a *= scale;
                if (causal && j > i) a = -INFINITY;
                s[jj] = a;
                if (a > tmax) tmax = a;
            }
            float mn = m > tmax ? m : tmax;
            float alpha = expf(m - mn);          /* m = -inf on the first tile -> alpha = 0 */
            for (int64_t d = 0; d < D; ++d) acc[d] *= alpha;
            l *= alpha;
            for (int64_t jj = 0; jj < jn; ++jj) {
                float p = expf(s[jj] - mn);
                l += p;                           /* the row sum uses the f32 P */
                float pb = round_bf16(p);         /* P is rounded to bf16 for the PV product */
                if (pb != 0.0f) {
                    const uint16_t* vr = v + (bh * N + j0 + jj) * D;
                    for (int64_t d = 0; d < D; ++d) acc[d] += pb * bf16_to_f32(vr[d]);
                }
            }
            m = mn;
        }
        for (int64_t d = 0; d < D; ++d) o_bf16[row * D + d] = f32_to_bf16(acc[d] / l);
        if (lse) lse[row] = logf(l) + m;
        free(acc); free(s);
    }
}

/* ----------------------------------------------------------- GQA decode -- */

/* One query token per sequence.  q: bf16 [B,Hq,1,D]; k,v: bf16 [B,Hkv,L,D]
 * (kv_stride = allocated rows per (b, kv-head), >= L: the preallocated cache);
 * q-head h reads kv-head h / (Hq/Hkv)  (repeat_interleave along the head axis).
 * The L positions are cut into num_splits contiguous chunks; each chunk produces
 * an un-normalised f32 partial (O_s, m_s, l_s); the merge is
 *   m = max m_s ; l = sum l_s e^{m_s-m} ; O = sum O_s e^{m_s-m} / l ; LSE = ln l + m.
 * o_bf16: bf16 [B,Hq,1,D]; lse: f32 [B,Hq] (may be NULL). */
void oracle_gqa_decode(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                       uint16_t* o_bf16, float* lse,
                       int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t D,
                       int64_t kv_stride, float scale, int64_t num_splits) {
    if (num_splits < 1) num_splits = 1;
    int64_t rep = Hq / Hkv;
    int64_t chunk = (L + num_splits - 1) / num_splits;
    #pragma omp parallel for schedule(dynamic)
    for (int64_t bh = 0; bh < B * Hq; ++bh) {
        int64_t b = bh / Hq, h = bh % Hq, g = h / rep;
        const uint16_t* qr = q + bh * D;
        const uint16_t* kb = k + (b * Hkv + g) * kv_stride * D;
        const uint16_t* vb = v + (b * Hkv + g) * kv_stride * D;
        float* po = (float*)calloc((size_t)(num_splits * D), sizeof(float));
        float* pm = (float*)malloc(sizeof(float) * (size_t)num_splits);
        float* pl = (float*)malloc(sizeof(float) * (size_t)num_splits);
        for (int64_t s = 0; s < num_splits; ++s) {
            int64_t j0 = s * chunk, j1 = j0 + chunk < L ? j0 + chunk : L;
            float m = -INFINITY, l = 0.0f;
            float* acc = po + s * D;
            for (int64_t j = j0; j < j1; ++j) {
                float a = 0.0f;
                for (int64_t d = 0; d < D; ++d) a += bf16_to_f32(qr[d]) * bf16_to_f32(kb[j * D + d]);
                a *= scale;
                float mn = m > a ? m : a;
                float alpha = expf(m - mn);
                float p = expf(a - mn);
                l = l * alpha + p;
                float pb = round_bf16(p);
                for (int64_t d = 0; d < D; ++d) acc[d] = acc[d] * alpha + pb * bf16_to_f32(vb[j * D + d]);
                m = mn;
            }
            pm[s] = m; pl[s] = l;
        }
        float m = -INFINITY;
        for (int64_t s = 0; s < num_splits; ++s) if (pm[s] > m) m = pm[s];
        float l = 0.0f;
        for (int64_t s = 0; s < num_splits; ++s) if (pl[s] > 0.0f) l += pl[s] * expf(pm[s] - m);
        for (int64_t d = 0; d < D; ++d) {
            float a = 0.0f;
            for (int64_t s = 0; s < num_splits; ++s) if (pl[s] > 0.0f) a += po[s * D + d] * expf(pm[s] - m);
            o_bf16[bh * D + d] = f32_to_bf16(a / l);
        }
        if (lse) lse[bh] = logf(l) + m;
        free(po); free(pm); free(pl);
    }
}

/* ------------------------------------------------------------------ GEMM -- */

/* C[m,n] = bf16( sum_k f32(A[m,k]) * f32(B[k,n]) ), f32 accumulation in k order.
 * A: bf16 [M,K] row-major.  trans_b == 0: B is [K,N] row-major ("NN");
 * trans_b != 0: B is [N,K] row-major ("NT", C = A B^T). */
void oracle_gemm_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c,
                      int64_t M, int64_t N, int64_t K, int trans_b) {
    #pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        float* row = (float*)calloc((size_t)N, sizeof(float));
        if (!trans_b) {
            for (int64_t kk = 0; kk < K; ++kk) {
                float av = bf16_to_f32(a[m * K + kk]);
                const uint16_t* br = b + kk * N;
                for (int64_t n = 0; n < N; ++n) row[n] += av * bf16_to_f32(br[n]);
            }
        } else {
            for (int64_t n = 0; n < N; ++n) {
                float acc = 0.0f;
                for (int64_t kk = 0; kk < K; ++kk) acc += bf16_to_f32(a[m * K + kk]) * bf16_to_f32(b[n * K + kk]);
                row[n] = acc;
            }
        }
        for (int64_t n = 0; n < N; ++n) c[m * N + n] = f32_to_bf16(row[n]);
        free(row);
    }
}

/* C[m,n] = bf16( scale_a*scale_b * sum_k e4m3(Aq[m,k]) * e4m3(Bq[k,n]) ), f32 accumulation,
 * the scalar applied once in the epilogue.  c_f32 (optional) receives the un-rounded value. */
void oracle_gemm_fp8(const uint8_t* aq, const uint8_t* bq, uint16_t* c, float* c_f32,
                     int64_t M, int64_t N, int64_t K,
                     float scale_a, float scale_b, int trans_b) {
    float lut[256];
    for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3_decode((uint8_t)i);
    float sc = scale_a * scale_b;
    #pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        float* row = (float*)calloc((size_t)N, sizeof(float));
        if (!trans_b) {
            for (int64_t kk = 0; kk < K; ++kk) {
                float av = lut[aq[m * K + kk]];
                const uint8_t* br = bq + kk * N;
                for (int64_t n = 0; n < N; ++n) row[n] += av * lut[br[n]];
            }
        } else {
            for (int64_t n = 0; n < N; ++n) {
                float acc = 0.0f;
                for (int64_t kk = 0; kk < K; ++kk) acc += lut[aq[m * K + kk]] * lut[bq[n * K + kk]];
                row[n] = acc;
            }
        }
        for (int64_t n = 0; n < N; ++n) {
            float r = row[n] * sc;
            if (c) c[m * N + n] = f32_to_bf16(r);
            if (c_f32) c_f32[m * N + n] = r;
        }
        free(row);
    }
}

/* ------------------------------------------------------- rotary / layernorm -- */

/* x, y: [B,S,H,D] as f32 (is_bf16 = 0) or bf16 bit patterns (is_bf16 = 1); cos, sin f32 [S, D/2].
 * Products and sums are single f32 operations in the order of the reference expression. */
void oracle_rope(const void* x, const float* cosp, const float* sinp, void* y,
                 int64_t B, int64_t S, int64_t H, int64_t D, int is_bf16) {
    const int64_t h = D / 2;
    for (int64_t row = 0; row < B * S * H; ++row) {
        const int64_t s = (row / H) % S;
        for (int64_t i = 0; i < h; ++i) {
            float x1, x2;
            if (is_bf16) {
                x1 = bf16_to_f32(((const uint16_t*)x)[row * D + i]);
                x2 = bf16_to_f32(((const uint16_t*)x)[row * D + h + i]);
            } else {
                x1 = ((const float*)x)[row * D + i];
                x2 = ((const float*)x)[row * D + h + i];
            }
            const float c = cosp[s * h + i], sn = sinp[s * h + i];
            volatile float a = x1 * c, b = x2 * sn, d = x1 * sn, e = x2 * c;   /* no fused multiply-add */
            const float y1 = a - b, y2 = d + e;
            if (is_bf16) {
                ((uint16_t*)y)[row * D + i] = f32_to_bf16(y1);
                ((uint16_t*)y)[row * D + h + i] = f32_to_bf16(y2);
            } else {
                ((float*)y)[row * D + i] = y1;
                ((float*)y)[row * D + h + i] = y2;
            }
        }
    }
}

/* x, residual, out, out_resid: bf16 bit patterns [rows, d]; weight, bias: bf16 [d]. */
void oracle_layernorm_residual(const uint16_t* x, const uint16_t* residual, const uint16_t* weight,
                               const uint16_t* bias, uint16_t* out, uint16_t* out_resid,
                               int64_t rows, int64_t d, double eps) {
    #pragma omp parallel for
    for (int64_t r = 0; r < rows; ++r) {
        double sum = 0.0;
        for (int64_t i = 0; i < d; ++i) {
            const uint16_t v = f32_to_bf16(bf16_to_f32(x[r * d + i]) + bf16_to_f32(residual[r * d + i]));
            out_resid[r * d + i] = v;
            sum += (double)bf16_to_f32(v);
        }
        const double mean = sum / (double)d;
        double sq = 0.0;
        for (int64_t i = 0; i < d; ++i) {
            const double c = (double)bf16_to_f32(out_resid[r * d + i]) - mean;
            sq += c * c;
        }
        const double inv = 1.0 / sqrt(sq / (double)d + eps);
        for (int64_t i = 0; i < d; ++i) {
            const double v = ((double)bf16_to_f32(out_resid[r * d + i]) - mean) * inv *
                             (double)bf16_to_f32(weight[i]) + (double)bf16_to_f32(bias[i]);
            out[r * d + i] = f32_to_bf16((float)v);
        }
    }
}

int oracle_num_threads(void) {
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}
