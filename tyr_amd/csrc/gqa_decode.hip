// GQA decode attention for gfx950: one query token per sequence, split-KV first pass plus an
// LSE-combine second pass.  HBM-bound: every K and V byte is read exactly once, straight from
// global memory into MFMA operand registers (no LDS staging), 16 bytes per lane per load.
//
// Contract of the reference: cc/src/tyr.cpp:4100-4133 (repeat_interleave of K/V along the head
// axis, then scaled_dot_product_attention with q_len = 1, is_causal = false); the Hq/Hkv query
// heads that share a kv head are packed into one MFMA tile as in
// Tyr/GPU/Kernels/FlashAttn3.lean:535-624; softmax order of Tyr/GPU/Codegen/Macros.lean:121-163;
// partial results are merged with the online-softmax algebra
//   m = max m_s ; l = sum l_s 2^(m_s-m) ; O = sum O_s 2^(m_s-m) / l ; LSE = ln l + m ln 2.
//
// First pass.  grid = splits * B*Hkv workgroups (the splits of a group adjacent), 8 waves per workgroup; the waves take the 32-row steps of
// the split in turn, each with the 16x16x32 bf16 MFMA:
//   S^T (16 kv x 16 q)  = K rows (row operand: lane l holds row l%16, 8 d at 32i + 8(l/16))
//                         x Q^T (column operand, zero beyond the G = Hq/Hkv real heads)
//   O^T_j (16 d x 16 q) += V^T (row operand) x P^T (column operand),  j = 0..7
// V is loaded row-major with full 256-byte rows per 16 lanes (lane x = l%16 takes columns
// 8x..8x+7 of 8 rows), transposed 8x8 in registers, and product j then covers d = 8x + j.
// The 8 rows a lane group takes are exactly the kv rows whose probabilities the S^T accumulator
// layout leaves in that lane group, so P^T needs no cross-lane movement.
// The waves merge through LDS and the workgroup writes one f32 partial (O, m, l) per split -- or,
// when there is a single split, the final bf16 O and LSE (no second pass).
#include "common.hpp"
#include "launch.hpp"

namespace tyr {

namespace dec {
constexpr int STEP = 32, QPAD = 16;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

template <int D>
struct Buf {
    u32x4 k[2][D / 32];   // [T][i]: row 16T + x, d = 32i + 8g + [0,8)
    u32x4 v[8];           // [p]  : row 16(p/4) + 4g + p%4, d = 8(x mod D/8) + [0,8)
};
}  // namespace dec

// WAVES waves per workgroup share one split.  With a single split (S == 1) the workgroup writes
// the final bf16 O and LSE itself and the second pass is skipped.
// D = 64: a V row is 8 pieces, so lanes x >= 8 repeat the loads of lanes x - 8 (same cache lines, no
// extra traffic) and rows 8..15 of every O^T MFMA tile (lane groups g >= 2) are unused.
template <int WAVES, int D>
__global__ __launch_bounds__(64 * WAVES) void gqa_decode_split_kernel(
    const uint16_t* __restrict__ Q, const uint16_t* __restrict__ Kp, const uint16_t* __restrict__ Vp,
    float* __restrict__ part_o, float* __restrict__ part_m, float* __restrict__ part_l,
    uint16_t* __restrict__ O, float* __restrict__ LSE,
    int Hq, int Hkv, int G, int L, long kv_stride, int S, int chunk, float scale_log2,
    const int* __restrict__ kv_lens, int window) {
    using namespace dec;
    constexpr int THREADS = 64 * WAVES;
    extern __shared__ __attribute__((aligned(16))) float smem[];   // [WAVES][G][D] O, then [WAVES][QPAD] m, l

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int x = lane & 15, g = lane >> 4;
    // one-dimensional grid, the splits of a (batch, kv head) group adjacent: any number of groups fits
    const int split = (int)(blockIdx.x % (unsigned)S);
    const int bg = (int)(blockIdx.x / (unsigned)S);   // b * Hkv + kv head
    const int b = bg / Hkv, kvh = bg % Hkv;

    const uint16_t* Kb = Kp + (size_t)bg * kv_stride * D;
    const uint16_t* Vb = Vp + (size_t)bg * kv_stride * D;

    // Per-sequence length (a padding mask over the cache tail) and sliding window: this sequence
    // attends to cache rows [lo, L).  A length of zero (an empty sequence) gives O = 0, LSE = -inf.
    if (kv_lens != nullptr) L = max(0, min(L, kv_lens[b]));
    const int lo = window > 0 ? max(0, L - window) : 0;
    const int c0 = lo + split * chunk;
    const int c1 = min(L, c0 + chunk);
    // The waves of a workgroup take the 32-row steps of its chunk in turn (wave w: steps w, w + 8, ...),
    // so the workgroup reads K and V as one contiguous front: +2 % over a contiguous slice per wave.
    const int r0 = c0 + w * STEP;
    const int r1 = c1;
    constexpr int SST = WAVES * STEP;           // rows from one step of a wave to its next
    const int nsteps = r1 > r0 ? (r1 - r0 + SST - 1) / SST : 0;

    // Q^T operand: column x = query head kvh*G + x (zero for x >= G)
    constexpr int KI = D / 32;                  // MFMA k-steps of a score tile
    bf16x8 qf[KI];
    {
        const uint16_t* qp = Q + ((size_t)b * Hq + (size_t)kvh * G + min(x, G - 1)) * D + g * 8;
#pragma unroll
        for (int i = 0; i < KI; ++i) {
            u32x4 v = ld_global_16(qp + i * 32);
            if (x >= G) v = u32x4{0, 0, 0, 0};
            qf[i] = __builtin_bit_cast(bf16x8, v);
        }
    }

    f32x4 oacc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) oacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m2 = -INFINITY, lsum = 0.0f;

    auto load = [&](Buf<D>& bf, int row0) {
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const int row = min(row0 + 16 * T + x, L - 1);
            const uint16_t* kp = Kb + (size_t)row * D + g * 8;
#pragma unroll
            for (int i = 0; i < KI; ++i) bf.k[T][i] = ld_global_16_nt(kp + i * 32);
        }
#pragma unroll
        for (int p = 0; p < 8; ++p) {
            const int row = min(row0 + 16 * (p >> 2) + 4 * g + (p & 3), L - 1);
            bf.v[p] = ld_global_16_nt(Vb + (size_t)row * D + (x & (D / 8 - 1)) * 8);
        }
    };

    auto compute = [&](const Buf<D>& bf, int row0) {
        f32x4 sacc[2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            sacc[T] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < KI; ++i)
                sacc[T] = mfma_16x16x32_bf16(__builtin_bit_cast(bf16x8, bf.k[T][i]), qf[i], sacc[T]);
        }
        // register rr of sub-tile T is kv row row0 + 16T + 4g + rr
        if (row0 + STEP > r1) {
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr)
                    if (row0 + 16 * T + 4 * g + rr >= r1) sacc[T][rr] = -INFINITY;
        }
        float mx = sacc[0][0];
#pragma unroll
        for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) mx = fmaxf(mx, sacc[T][rr]);
        mx = max_xor32(max_xor16(mx));
        const float m2new = fmaxf(m2, mx * scale_log2);
        const float alpha = fast_exp2(m2 - m2new);
        if (__builtin_amdgcn_ballot_w64(m2new > m2) != 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j) oacc[j] *= alpha;
        }
        m2 = m2new;
        float pv[8];
        float psum = 0.0f;
#pragma unroll
        for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                pv[4 * T + rr] = fast_exp2(fmaf(sacc[T][rr], scale_log2, -m2new));
                psum += pv[4 * T + rr];
            }
        lsum = lsum * alpha + psum;
        u32x4 pk;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) pk[jj] = pack_bf16(pv[2 * jj], pv[2 * jj + 1]);
        const bf16x8 pfrag = __builtin_bit_cast(bf16x8, pk);

        u32x4 vt[8];
        transpose8x8_b16(bf.v, vt);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            oacc[j] = mfma_16x16x32_bf16(__builtin_bit_cast(bf16x8, vt[j]), pfrag, oacc[j]);
    };

    // the first K / V rows are requested before Q is waited for (loads return in order: waiting for
    // the older Q does not wait for them)
    Buf<D> b0, b1;
    if (nsteps > 0) load(b0, r0);
#pragma unroll
    for (int i = 0; i < KI; ++i) pin_registers(qf[i]);
    for (int st = 0; st < nsteps; st += 2) {
        if (st + 1 < nsteps) load(b1, r0 + (st + 1) * SST);
        compute(b0, r0 + st * SST);
        if (st + 1 < nsteps) {
            if (st + 2 < nsteps) load(b0, r0 + (st + 2) * SST);
            compute(b1, r0 + (st + 1) * SST);
        }
    }

    // ---- merge the waves through LDS.  oacc[j][rr] is O^T[d = 32g + 8rr + j][q = x].
    float* so = smem;                              // [WAVES][G][D]
    float* sm = smem + WAVES * G * D;              // [WAVES][QPAD]
    float* sl = sm + WAVES * QPAD;                 // [WAVES][QPAD]
    const float ltot = sum_xor32(sum_xor16(lsum));
    if (x < G && 32 * g < D) {
        float* dst = so + ((size_t)w * G + x) * D + 32 * g;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            *reinterpret_cast<f32x4*>(dst + 8 * rr) = f32x4{oacc[0][rr], oacc[1][rr], oacc[2][rr], oacc[3][rr]};
            *reinterpret_cast<f32x4*>(dst + 8 * rr + 4) = f32x4{oacc[4][rr], oacc[5][rr], oacc[6][rr], oacc[7][rr]};
        }
    }
    if (x < G && g == 0) { sm[w * QPAD + x] = m2; sl[w * QPAD + x] = ltot; }
    __syncthreads();

    for (int idx = t; idx < G * D; idx += THREADS) {
        const int qh = idx / D, d = idx % D;
        float m = -INFINITY;
#pragma unroll
        for (int ww = 0; ww < WAVES; ++ww) m = fmaxf(m, sm[ww * QPAD + qh]);
        float o = 0.0f, l = 0.0f;
        if (m > -INFINITY) {
#pragma unroll
            for (int ww = 0; ww < WAVES; ++ww) {
                const float wgt = fast_exp2(sm[ww * QPAD + qh] - m);
                o += so[((size_t)ww * G + qh) * D + d] * wgt;
                l += sl[ww * QPAD + qh] * wgt;
            }
        }
        const size_t head = (size_t)b * Hq + (size_t)kvh * G + qh;
        if (S == 1) {
            O[head * D + d] = (uint16_t)(pack_bf16(l > 0.0f ? o / l : 0.0f, 0.0f) & 0xffffu);
            if (d == 0 && LSE != nullptr) LSE[head] = l > 0.0f ? logf(l) + m * LN2 : -INFINITY;
        } else {
            const size_t ph = head * S + split;
            part_o[ph * D + d] = o;
            if (d == 0) { part_m[ph] = m; part_l[ph] = l; }
        }
    }
}

// Second pass: one workgroup of D threads per (batch, query head).
template <int D>
__global__ __launch_bounds__(D) void gqa_decode_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_m, const float* __restrict__ part_l,
    uint16_t* __restrict__ O, float* __restrict__ LSE, int S) {
    using namespace dec;
    const int bh = blockIdx.x, d = threadIdx.x;
    const float* pm = part_m + (size_t)bh * S;
    const float* pl = part_l + (size_t)bh * S;
    const float* po = part_o + (size_t)bh * S * D + d;
    float m = -INFINITY;
#pragma unroll 8
    for (int s = 0; s < S; ++s) m = fmaxf(m, pm[s]);
    // The loads of a partial do not depend on its weight, so eight splits are in flight at a time
    // (an empty split's O is never written: it is read and discarded, not multiplied).
    float o = 0.0f, l = 0.0f;
#pragma unroll 8
    for (int s = 0; s < S; ++s) {
        const float ms = pm[s];
        const float os = po[(size_t)s * D], ls = pl[s];
        const bool live = ms > -INFINITY;
        const float wgt = live ? fast_exp2(ms - m) : 0.0f;
        o += live ? os * wgt : 0.0f;
        l += live ? ls * wgt : 0.0f;
    }
    const float res = l > 0.0f ? o / l : 0.0f;    // every split empty: the sequence has no keys
    // pairs of threads pack two bf16 into one dword
    const float nb = __shfl_down(res, 1);
    if ((d & 1) == 0) reinterpret_cast<uint32_t*>(O + (size_t)bh * D)[d >> 1] = pack_bf16(res, nb);
    if (LSE != nullptr && d == 0) LSE[bh] = l > 0.0f ? logf(l) + m * LN2 : -INFINITY;
}

int launch_gqa_decode(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                      int Hq, int Hkv, int L, int D, int64_t kv_stride, float scale, int num_splits,
                      void* workspace, const int* kv_lens, int window, hipStream_t stream) {
    using namespace dec;
    constexpr int WAVES = 8;
    const int G = Hq / Hkv;
    const int S = num_splits;
    const int span = window > 0 ? (window < L ? window : L) : L;     // longest range any sequence reads
    int chunk = (span + S - 1) / S;
    chunk = (chunk + STEP - 1) / STEP * STEP;

    float* part_o = static_cast<float*>(workspace);
    float* part_m = part_o + (size_t)B * Hq * S * D;
    float* part_l = part_m + (size_t)B * Hq * S;

    const size_t lds = (size_t)(WAVES * G * D + 2 * WAVES * QPAD) * sizeof(float);
    dim3 grid((unsigned)((size_t)S * B * Hkv)), block(64 * WAVES);
#define TYR_DEC_LAUNCH(DD)                                                                           \
    do {                                                                                             \
        static const hipError_t attr = hipFuncSetAttribute(                                          \
            reinterpret_cast<const void*>(&gqa_decode_split_kernel<WAVES, DD>),                      \
            hipFuncAttributeMaxDynamicSharedMemorySize,                                              \
            (WAVES * QPAD * DD + 2 * WAVES * QPAD) * (int)sizeof(float));                            \
        if (attr != hipSuccess) return -1;                                                           \
        hipLaunchKernelGGL((gqa_decode_split_kernel<WAVES, DD>), grid, block, lds, stream,           \
                           static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k),         \
                           static_cast<const uint16_t*>(v), part_o, part_m, part_l,                  \
                           static_cast<uint16_t*>(o), lse, Hq, Hkv, G, L, (long)kv_stride, S, chunk, \
                           scale * LOG2E, kv_lens, window);                                          \
        if (hipGetLastError() != hipSuccess) return -1;                                              \
        if (S > 1) {                                                                                 \
            hipLaunchKernelGGL(gqa_decode_combine_kernel<DD>, dim3((unsigned)(B * Hq)), dim3(DD), 0, \
                               stream, part_o, part_m, part_l, static_cast<uint16_t*>(o), lse, S);   \
            if (hipGetLastError() != hipSuccess) return -1;                                          \
        }                                                                                            \
    } while (0)
    if (D == 128) TYR_DEC_LAUNCH(128); else TYR_DEC_LAUNCH(64);
#undef TYR_DEC_LAUNCH
    return 0;
}

}  // namespace tyr
