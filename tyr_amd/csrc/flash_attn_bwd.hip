// Flash-attention backward for gfx950 (bf16 in, f32 accumulation, bf16 dQ / dK / dV).
//
// Arithmetic contract of the reference (Tyr/GPU/Kernels/MhaH100.lean):
//   :197-232  backward prep      delta[i] = sum_d dO[i,d] * O[i,d]
//   :234-344  backward           S = Q K^T * scale ; P = exp(S - lse) ; dP = dO V^T ;
//                                dS = P o (dP - delta) ; dV += bf16(P)^T dO ;
//                                dK += bf16(dS)^T Q * scale ; dQ += bf16(dS) K * scale
// (expected values in the reference's runner come from autograd of scaled_dot_product_attention,
// Examples/GPU/RunMhaH100.lean:56-64).  exp is evaluated as exp2 with log2(e) folded into the
// scale and into the saved log-sum-exp.  causal: key j visible to query i iff j <= i.
//
// Two kernels, no atomics, every output written once (results are deterministic):
//
//  1. flash_attn_bwd_dq_kernel: one workgroup = 128 query rows (4 waves x 32 rows), keys/values
//     stream through LDS in tiles of 64 rows exactly as in the forward kernel.  Products are
//     computed transposed so that every lane owns one query column:
//        S^T  (64 kv x 32 q) = K_tile x Q^T       dP^T (64 kv x 32 q) = V_tile x dO^T
//        dQ^T (D x 32 q)    += K_tile^T x dS^T
//     so lse and delta are per-lane scalars and dS^T is already in the register slots the third
//     product wants as its column operand.  The prologue also computes delta (each wave holds its
//     dO rows and reads its O rows once) and writes (lse * log2 e, delta) pairs to the workspace
//     for the second kernel; rows of the padding up to a multiple of 128 get (+inf, 0), which
//     makes their probabilities exactly zero.
//
//  2. flash_attn_bwd_dkv_kernel: one workgroup = 128 key rows (4 waves x 32 rows, K and V
//     fragments of those rows live in registers), queries / dO stream through LDS in tiles of 64
//     rows, four stages deep.  Every lane owns one key column:
//        S  (32 q x 32 kv) = Q_tile x K_w^T        dP (32 q x 32 kv) = dO_tile x V_w^T
//        dV^T (D x 32 kv) += dO_tile^T x P         dK^T (D x 32 kv) += Q_tile^T x dS
//     with lse / delta of the 16 query rows a lane holds read from the staged pairs.
//
// Both recompute S (7 matrix products for an algorithm that needs 5): the price of writing dQ
// without a float atomic accumulation buffer and a conversion pass.
//
// LDS tiles are row-major with 16-byte chunks XOR-swizzled by a function of the row that is
// conflict-free both for row fragments (16-byte reads, lane = row) and for transposed fragments
// (ds_read_b64_tr_b16 over 4 rows x 64 bytes per lane-group pair).
#include <limits.h>
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace tyr {

namespace fab {
constexpr int THREADS = 256;
constexpr float LOG2E = 1.4426950408889634f;

// chunk index within a row -> stored chunk index.  The mask is a bijection of (row mod 16) [of
// ((row / 2) mod 8) for 128-byte rows], so 16 consecutive rows put one logical chunk on 16
// different bank groups; its upper bits follow row mod 4, which spreads the 4 rows a lane group
// of the transposing read touches over the 4 64-byte quarters of the bank space.
template <int D> __device__ __forceinline__ int swz(int row, int c) {
    return D == 128 ? (c ^ (((row & 3) << 2) | ((row >> 2) & 3)))
                    : (c ^ ((((row >> 1) & 1) << 2) | ((row >> 2) & 3)));
}

template <int D>
struct CfgQ {                                       // dQ kernel
    static constexpr int BM = 128, BN = 64;
    static constexpr int ROW = D * 2, KCH = D / 8;
    static constexpr int TILE = BN * ROW;
    static constexpr int V_BASE = 2 * TILE;         // K stage 0, K stage 1, V stage 0, V stage 1
    static constexpr int LDS = 4 * TILE;
    static constexpr int PT = BN * KCH / THREADS;   // 16-byte chunks per thread per tile
    static constexpr int KSTEPS = D / 16, DT = D / 32;
};

template <int D>
struct CfgK {                                       // dK / dV kernel
    static constexpr int BNK = 128, BQ = 64, NST = 4;   // NST must stay a power of two
    static constexpr int ROW = D * 2, KCH = D / 8;
    static constexpr int TILE = BQ * ROW;
    static constexpr int STAT = 1024;               // 64 (lse2, delta) pairs + slack of one load
    static constexpr int STAGE = 2 * TILE + STAT;   // Q tile, dO tile, pairs
    static constexpr int LDS = NST * STAGE;
    static constexpr int PT = BQ * KCH / THREADS;
    static constexpr int KSTEPS = D / 16, DT = D / 32;
    static constexpr int LOADS_PER_TILE = 2 * PT + 1;
};

__device__ __forceinline__ float dot8_bf16(u32x4 a, u32x4 b) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) s += bf16_lo(a[i]) * bf16_lo(b[i]) + bf16_hi(a[i]) * bf16_hi(b[i]);
    return s;
}

// One wave's 32 columns x D rows accumulator (lane = column l%32, register e of tile dt <-> row
// 32 dt + 8(e/4) + 4(l/32) + e%4), scaled, written as bf16 rows of length D: out row = column.
// Goes through a private LDS scratch so the global stores are 16 bytes per lane along rows.
template <int D>
__device__ __forceinline__ void store_transposed_bf16(const f32x16 (&acc)[D / 32], float mul, unsigned char* scratch,
                                                      uint16_t* out_rows, int rows_valid, int lane) {
    constexpr int SROW = D * 2 + 16;
    const int r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int dt = 0; dt < D / 32; ++dt) {
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
            u32x2 v;
            v.x = pack_bf16(acc[dt][4 * q4 + 0] * mul, acc[dt][4 * q4 + 1] * mul);
            v.y = pack_bf16(acc[dt][4 * q4 + 2] * mul, acc[dt][4 * q4 + 3] * mul);
            *reinterpret_cast<u32x2*>(scratch + r * SROW + (dt * 32 + q4 * 8 + g * 4) * 2) = v;
        }
    }
    constexpr int CH = D / 8;
    constexpr int RPI = 64 / CH;
#pragma unroll
    for (int k = 0; k < 32 / RPI; ++k) {
        const int row = lane / CH + RPI * k;
        const u32x4 v = *reinterpret_cast<const u32x4*>(scratch + row * SROW + (lane % CH) * 16);
        if (row < rows_valid) st_global_16(out_rows + (size_t)row * D + (lane % CH) * 8, v);
    }
}
}  // namespace fab

// ------------------------------------------------------------------------------------------
// dQ (and the (lse2, delta) pairs)
// EXT adds the per-sequence key length and the sliding window (same rule as the forward kernel);
// G = query heads per kv head.
template <int D, bool CAUSAL, bool EXT>
__global__ __launch_bounds__(fab::THREADS, 2) void flash_attn_bwd_dq_kernel(
    const uint16_t* __restrict__ Q, const uint16_t* __restrict__ Kp, const uint16_t* __restrict__ Vp,
    const uint16_t* __restrict__ O, const uint16_t* __restrict__ dO, const float* __restrict__ LSE,
    uint16_t* __restrict__ dQ, float2* __restrict__ stats, int BH, int N, int ntq, float scale,
    float scale_log2, int Hq, int G, int window, const int* __restrict__ kv_lens,
    const uint8_t* __restrict__ key_mask, int pair) {
    using namespace fab;
    using C = CfgQ<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, g = lane >> 5;

    // With `pair` (causal) a workgroup handles query tile ntq-1-tr and then tile tr (equal work
    // for every workgroup, half as many of them).
    const int ntr = pair ? (ntq + 1) / 2 : ntq;
    int bh, tr, kvbh;
    {
        const int id = blockIdx.x;
        const int ngroups = BH / G;              // B * Hkv: the unit dealt to an XCD shares one K / V
        if ((ngroups & 7) == 0) {
            const int xcd = id & 7, slot = id >> 3;
            const int per_group = G * ntr;
            kvbh = (slot / per_group) * 8 + xcd;
            const int within = slot % per_group;
            tr = within / G;
            const int hkv = Hq / G;
            bh = (kvbh / hkv) * Hq + (kvbh % hkv) * G + within % G;
        } else {
            bh = id / ntr;
            tr = id % ntr;
            kvbh = (bh / Hq) * (Hq / G) + (bh % Hq) / G;
        }
    }
    const int npass = (pair && ntq - 1 - tr != tr) ? 2 : 1;
    for (int pass = 0; pass < npass; ++pass) {
    const int qt = CAUSAL ? (pass == 0 ? ntq - 1 - tr : tr) : tr;
    const int q0 = qt * C::BM;
    const int qw0 = q0 + w * 32;
    const size_t head_off = (size_t)bh * N * D;
    const uint16_t* Kh = Kp + (size_t)kvbh * N * D;
    const uint16_t* Vh = Vp + (size_t)kvbh * N * D;
    const int Nk = (EXT && kv_lens != nullptr) ? max(0, min(N, kv_lens[bh / Hq])) : N;
    const uint8_t* km = (EXT && key_mask != nullptr) ? key_mask + (size_t)(bh / Hq) * N : nullptr;
    const int kv_end = CAUSAL ? min(Nk, q0 + C::BM) : Nk;
    const int nkv_abs = max(1, (kv_end + C::BN - 1) / C::BN);   // a sequence without keys still walks one (fully masked) tile
    const int jbase = (EXT && window > 0) ? min(max(0, q0 - window + 1) / C::BN, nkv_abs - 1) : 0;
    const int nkv = nkv_abs - jbase;             // tiles are numbered from jbase below
    const int qpos = qw0 + r;

    // ---- this wave's Q^T and dO^T fragments (lane = query row, columns 16i + 8g + [0,8)),
    //      delta = dO . O and lse in log2 units
    bf16x8 qf[C::KSTEPS], dof[C::KSTEPS];
    float delta, lse2;
    {
        const int qrow = min(qpos, N - 1);
        const size_t off = head_off + (size_t)qrow * D + g * 8;
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i) {
            qf[i] = __builtin_bit_cast(bf16x8, ld_global_16(Q + off + i * 16));
            const u32x4 dv = ld_global_16(dO + off + i * 16);
            const u32x4 ov = ld_global_16(O + off + i * 16);
            dof[i] = __builtin_bit_cast(bf16x8, dv);
            part += dot8_bf16(dv, ov);
        }
        delta = part + xor32(part);
        lse2 = LSE[(size_t)bh * N + qrow] * LOG2E;
        if (EXT && lse2 == -INFINITY) lse2 = INFINITY;      // a row that saw no key: every probability is 0
        if (g == 0) {
            const size_t npad = (size_t)ntq * C::BM;
            stats[(size_t)bh * npad + qpos] = qpos < N ? make_float2(lse2, delta) : make_float2(INFINITY, 0.0f);
        }
    }

    // ---- K / V tile loaders (global memory straight into LDS, swizzle applied on the global side)
    const uint32_t head_bytes = (uint32_t)N * D * 2u;
    const u32x4 k_rsrc = make_raw_rsrc(Kh, head_bytes);
    const u32x4 v_rsrc = make_raw_rsrc(Vh, head_bytes);
    constexpr int ROWS_PER_INST = 1024 / C::ROW;
    int g_voff[C::PT];
#pragma unroll
    for (int m = 0; m < C::PT; ++m) {
        const int row = (w * C::PT + m) * ROWS_PER_INST + lane / C::KCH;
        g_voff[m] = row * C::ROW + swz<D>(row, lane % C::KCH) * 16 - 1024 * m;   // request m carries 1024 m as its immediate offset
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t wave_dst = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)w * C::PT * 1024u);
    auto issue_kv = [&](int stage, int j0) {
        const uint32_t dst = wave_dst + (uint32_t)stage * C::TILE;
        load_global_to_lds_16xN<C::PT>(k_rsrc, dst, g_voff, j0 * C::ROW);
        load_global_to_lds_16xN<C::PT>(v_rsrc, dst + C::V_BASE, g_voff, j0 * C::ROW);
    };

    // row fragment (sub-tile T, k-step i): row 32T + r, chunk 2i + g
    int row_off[C::KSTEPS];
#pragma unroll
    for (int i = 0; i < C::KSTEPS; ++i) row_off[i] = r * C::ROW + swz<D>(r, 2 * i + g) * 16;
    // transposed fragment (d tile dt; kv rows 16c + 8h + 4g + [0,4)): as a source lane of the
    // transposing read this lane points at row 4(b/2) + (lane%16)/4 (+8 for the second read),
    // 8 bytes at d = 32dt + 16(b&1) + 4(lane%4), b = lane/16.
    int tr_lo[C::DT], tr_hi[C::DT];
    {
        const int i16 = lane & 15, b16 = lane >> 4;
        const int row = 4 * (b16 >> 1) + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            const int dcol = 32 * dt + 16 * (b16 & 1) + 4 * (i16 & 3);
            tr_lo[dt] = row * C::ROW + swz<D>(row, dcol >> 3) * 16 + (dcol & 7) * 2;
            tr_hi[dt] = (row + 8) * C::ROW + swz<D>(row + 8, dcol >> 3) * 16 + (dcol & 7) * 2;
        }
    }

    f32x16 dq[C::DT];
#pragma unroll
    for (int i = 0; i < C::DT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) dq[i][e] = 0.0f;

    const int nkv_w = CAUSAL ? min(nkv, (qw0 + 31) / C::BN + 1 - jbase) : nkv;

    issue_kv(0, jbase * C::BN);
#pragma unroll
    for (int i = 0; i < C::KSTEPS; ++i) { pin_registers(qf[i]); pin_registers(dof[i]); }
    wait_vmcnt0();
    __syncthreads();

    for (int j = 0; j < nkv; ++j) {
        const int j0 = (jbase + j) * C::BN;
        if (j + 1 < nkv) issue_kv((j + 1) & 1, j0 + C::BN);
        if (j < nkv_w) {
            const unsigned char* Kt = lds + (j & 1) * C::TILE;
            const unsigned char* Vt = Kt + C::V_BASE;
            // The two 32-row sub-tiles of the tile are taken one after the other (scores, probabilities, dQ
            // products): only one sub-tile's scores are live, which leaves the registers the fragment read-ahead
            // needs; the other wave of the SIMD has matrix work while this one does its exponentials.
            f32x16 s[2], dp[2];
            bf16x8 dsf[4];
            // the tile's 64 key-mask bytes as one word (bit r set: kv row j0 + r is hidden): one byte per
            // lane and a ballot; a tile without hidden rows skips the masking
            uint64_t tile_hidden = 0;
            if (EXT && km != nullptr) tile_hidden = __builtin_amdgcn_ballot_w64(km[min(j0 + lane, N - 1)] == 0);
            const bool need_mask = (CAUSAL && (j0 + C::BN - 1 > qw0)) || (j0 + C::BN > Nk) ||
                                   (EXT && window > 0 && j0 < qw0 + 32 - window) || (EXT && tile_hidden != 0);
            // Fragments are read one k-step ahead of the products that take them, also across the phases of a tile (the
            // first fragments of a phase are requested under the last products of the phase before it), and the
            // scheduling barriers keep that order: left to itself the compiler, at its register limit, puts every read
            // right in front of its product and the wave waits out the LDS latency 48 times per tile.
            bf16x8 ka[2], va[2];                 // K / V row fragments of the scores phase
            bf16x4 lo[2], hi[2];                 // transposed K fragments of the dQ phase
            auto read_rows = [&](int T, int i, int slot) {
                ka[slot] = *reinterpret_cast<const bf16x8*>(Kt + row_off[i] + T * 32 * C::ROW);
                va[slot] = *reinterpret_cast<const bf16x8*>(Vt + row_off[i] + T * 32 * C::ROW);
            };
            auto read_transposed = [&](int T, int n, int slot) {      // n = (c - 2T) * DT + dt
                const int c = 2 * T + n / C::DT, dt = n % C::DT;
                lo[slot] = ds_read_tr16(Kt + tr_lo[dt] + c * 16 * C::ROW);
                hi[slot] = ds_read_tr16(Kt + tr_hi[dt] + c * 16 * C::ROW);
            };
            auto scores = [&](int T) {           // expects the fragments of k-step 0 in slot 0
#pragma unroll
                for (int e = 0; e < 16; ++e) { s[T][e] = 0.0f; dp[T][e] = 0.0f; }
#pragma unroll
                for (int i = 0; i < C::KSTEPS; ++i) {
                    if (i + 1 < C::KSTEPS) read_rows(T, i + 1, (i + 1) & 1);
                    else read_transposed(T, 0, 0);               // first fragment of this sub-tile's dQ phase
                    __builtin_amdgcn_sched_barrier(0);
                    s[T] = mfma_32x32x16_bf16(ka[i & 1], qf[i], s[T]);
                    dp[T] = mfma_32x32x16_bf16(va[i & 1], dof[i], dp[T]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            // mask (diagonal tiles, ragged tail), then dS^T = P^T o (dP^T - delta) packed into column-operand
            // slots (group c = 2T + sh holds registers 8sh .. 8sh+7 of sub-tile T).  Register e of sub-tile T
            // is kv row j0 + 32T + 8(e/4) + 4g + e%4.
            auto probabilities = [&](int T) {
                if (need_mask) {
                    const int lim = CAUSAL ? min(qpos, Nk - 1) : Nk - 1;
                    const int low = (EXT && window > 0) ? qpos - window + 1 : INT_MIN;
                    const int base = j0 + 4 * g;
                    const uint64_t hidden = tile_hidden >> (4 * g + 32 * T);      // shifted to this lane's rows
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int kv = base + 32 * T + 8 * (e >> 2) + (e & 3);
                        const bool off = kv > lim || (EXT && kv < low) || ((hidden >> (8 * (e >> 2) + (e & 3))) & 1u);
                        s[T][e] = off ? -INFINITY : s[T][e];
                    }
                }
#pragma unroll
                for (int sh = 0; sh < 2; ++sh) {
                    u32x4 pk;
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) {
                        const int e = 8 * sh + 2 * jj;
                        const float p0 = fast_exp2(fmaf(s[T][e], scale_log2, -lse2));
                        const float p1 = fast_exp2(fmaf(s[T][e + 1], scale_log2, -lse2));
                        pk[jj] = pack_bf16(p0 * (dp[T][e] - delta), p1 * (dp[T][e + 1] - delta));
                    }
                    dsf[2 * T + sh] = __builtin_bit_cast(bf16x8, pk);
                }
            };
            // dQ^T += K^T dS^T for the two 16-row groups of sub-tile T
            auto accumulate = [&](int T) {       // expects the transposed fragment 0 in slot 0
#pragma unroll
                for (int n = 0; n < 2 * C::DT; ++n) {
                    const int c = 2 * T + n / C::DT, dt = n % C::DT;
                    if (n + 1 < 2 * C::DT) read_transposed(T, n + 1, (n + 1) & 1);
                    else if (T == 0) read_rows(1, 0, 0);         // first fragments of the second sub-tile's scores
                    __builtin_amdgcn_sched_barrier(0);
                    const bf16x8 kt = __builtin_shufflevector(lo[n & 1], hi[n & 1], 0, 1, 2, 3, 4, 5, 6, 7);
                    dq[dt] = mfma_32x32x16_bf16(kt, dsf[c], dq[dt]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            };
            read_rows(0, 0, 0);
            scores(0);
            probabilities(0);
            accumulate(0);
            scores(1);
            probabilities(1);
            accumulate(1);
        }
        wait_vmcnt0();
        __syncthreads();
    }

    store_transposed_bf16<D>(dq, scale, lds + w * (32 * (D * 2 + 16)), dQ + head_off + (size_t)qw0 * D,
                             N - qw0, lane);
    __syncthreads();                             // the scratch is read; the stages may be refilled
    }
}

// ------------------------------------------------------------------------------------------
// dK, dV
// BHkv = batch * kv heads; the G query heads of a kv head are walked one after the other and
// accumulate into the same dK / dV (the gradient of repeat_interleave).  EXT as above; with it
// every step carries the mask instructions.
template <int D, bool CAUSAL, bool EXT>
__global__ __launch_bounds__(fab::THREADS, 1) void flash_attn_bwd_dkv_kernel(
    const uint16_t* __restrict__ Q, const uint16_t* __restrict__ Kp, const uint16_t* __restrict__ Vp,
    const uint16_t* __restrict__ dO, const float2* __restrict__ stats, uint16_t* __restrict__ dK,
    uint16_t* __restrict__ dV, int BHkv, int N, int ntk, int npad, float scale, float scale_log2,
    int Hq, int G, int window, const int* __restrict__ kv_lens, const uint8_t* __restrict__ key_mask) {
    using namespace fab;
    using C = CfgK<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, g = lane >> 5;

    int bh, kt;                           // bh indexes (batch, kv head)
    {
        const int id = blockIdx.x;
        if ((BHkv & 7) == 0) {
            const int xcd = id & 7, slot = id >> 3;
            bh = (slot / ntk) * 8 + xcd;
            kt = slot % ntk;              // causal: key tile 0 meets every query tile, so heavy first
        } else {
            bh = id / ntk;
            kt = id % ntk;
        }
    }
    const int n0 = kt * C::BNK;
    const int nw0 = n0 + w * 32;
    const int kvpos = nw0 + r;
    const size_t head_off = (size_t)bh * N * D;                       // of K, V, dK, dV
    const int hkv = Hq / G;
    const size_t qh0 = (size_t)(bh / hkv) * Hq + (size_t)(bh % hkv) * G;   // first query head of the group
    const int Nk = (EXT && kv_lens != nullptr) ? max(0, min(N, kv_lens[bh / hkv])) : N;
    // this lane's key is hidden from every query by the key mask
    const bool key_off = EXT && key_mask != nullptr && key_mask[(size_t)(bh / hkv) * N + min(kvpos, N - 1)] == 0;

    // ---- this wave's K and V rows as column operands (lane = key row, columns 16i + 8g + [0,8))
    bf16x8 kf[C::KSTEPS], vf[C::KSTEPS];
    {
        const size_t off = head_off + (size_t)min(kvpos, N - 1) * D + g * 8;
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i) {
            kf[i] = __builtin_bit_cast(bf16x8, ld_global_16(Kp + off + i * 16));
            vf[i] = __builtin_bit_cast(bf16x8, ld_global_16(Vp + off + i * 16));
        }
    }

    // ---- Q / dO / pair tile loaders
    // The G query heads of the group are adjacent in memory: one buffer covers them, a head is a
    // scalar offset.  (Rows past N of a head then alias the next head's first rows instead of
    // reading as zero; their pairs are (+inf, 0), so their probabilities are exactly 0 either way.)
    const uint32_t head_bytes = (uint32_t)N * D * 2u;
    const u32x4 q_rsrc = make_raw_rsrc(Q + qh0 * N * D, head_bytes * (uint32_t)G);
    const u32x4 do_rsrc = make_raw_rsrc(dO + qh0 * N * D, head_bytes * (uint32_t)G);
    const uint32_t stat_bytes = (uint32_t)npad * 8u;
    const u32x4 st_rsrc = make_raw_rsrc(stats + qh0 * npad, stat_bytes * (uint32_t)G);
    constexpr int ROWS_PER_INST = 1024 / C::ROW;
    int g_voff[C::PT];
#pragma unroll
    for (int m = 0; m < C::PT; ++m) {
        const int row = (w * C::PT + m) * ROWS_PER_INST + lane / C::KCH;
        g_voff[m] = row * C::ROW + swz<D>(row, lane % C::KCH) * 16 - 1024 * m;   // request m carries 1024 m as its immediate offset
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t wave_dst = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)w * C::PT * 1024u);
    const int nq = (N + C::BQ - 1) / C::BQ;
    // Tiles past the end are requested at an offset beyond the buffer (they read as zero), so that
    // every iteration issues the same number of loads and the wait count below stays constant.
    const int jq0 = CAUSAL ? n0 / C::BQ : 0;
    // with a window the last query that sees a key of this block is n0 + 127 + window - 1
    const int jq_end = (EXT && window > 0) ? min(nq, (n0 + C::BNK + window - 2) / C::BQ + 1) : nq;
    int hq = 0;                                      // query head of the group being walked
    auto issue_tile = [&](int stage, int jq) {
        const uint32_t dst = wave_dst + (uint32_t)stage * C::STAGE;
        const bool live = jq < jq_end;
        const int soff = live ? hq * (int)head_bytes + jq * C::BQ * C::ROW : (int)(head_bytes * (uint32_t)G);
        const int ssoff = live ? (hq * npad + jq * C::BQ) * 8 : (int)(stat_bytes * (uint32_t)G);
        load_global_to_lds_16xN<C::PT>(q_rsrc, dst, g_voff, soff);
        load_global_to_lds_16xN<C::PT>(do_rsrc, dst + C::TILE, g_voff, soff);
        // every wave requests the same kilobyte of pairs (identical bytes, one instruction)
        load_global_to_lds_16(st_rsrc, lds_base + (uint32_t)stage * C::STAGE + 2 * C::TILE, lane * 16, ssoff);
    };

    int row_off[C::KSTEPS];
#pragma unroll
    for (int i = 0; i < C::KSTEPS; ++i) row_off[i] = r * C::ROW + swz<D>(r, 2 * i + g) * 16;
    int tr_lo[C::DT], tr_hi[C::DT];
    {
        const int i16 = lane & 15, b16 = lane >> 4;
        const int row = 4 * (b16 >> 1) + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            const int dcol = 32 * dt + 16 * (b16 & 1) + 4 * (i16 & 3);
            tr_lo[dt] = row * C::ROW + swz<D>(row, dcol >> 3) * 16 + (dcol & 7) * 2;
            tr_hi[dt] = (row + 8) * C::ROW + swz<D>(row + 8, dcol >> 3) * 16 + (dcol & 7) * 2;
        }
    }

    f32x16 dk[C::DT], dv[C::DT];
#pragma unroll
    for (int i = 0; i < C::DT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) { dk[i][e] = 0.0f; dv[i][e] = 0.0f; }

    const int ntile = jq_end - jq0;
    const int nsub = 2 * ntile;                       // 32-row sub-tiles, numbered from the block's first tile
    // First sub-tile with a visible (query, key) pair for this wave.  Causal: the block's first
    // tile starts at query n0 and the wave's keys at n0 + 32w, so sub-tile w is the wave's diagonal
    // one (the only partially masked one); earlier sub-tiles are skipped.
    const int u0 = CAUSAL ? w : 0;

    // LDS addresses.  Inside the pipeline the stage and the sub-tile of every access are
    // compile-time constants, so an address is a per-lane base register plus an immediate; the
    // immediate field holds 16 bits, hence a second set of bases for stages 2 and 3.
    // The bases are made opaque to the compiler, which would otherwise recompute each of them
    // (LDS symbol + offset) next to every use.
    typedef __attribute__((address_space(3))) const unsigned char* lds_cptr;
    auto opaque = [&](int off) {
        uint32_t a = lds_base + (uint32_t)off;
        asm volatile("" : "+v"(a));
        return (lds_cptr)(uintptr_t)a;
    };
    lds_cptr rowp[2][C::KSTEPS], trlo[2][C::DT], trhi[2][C::DT], statp[2];
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i) rowp[hh][i] = opaque(row_off[i] + hh * 2 * C::STAGE);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            trlo[hh][dt] = opaque(tr_lo[dt] + hh * 2 * C::STAGE);
            trhi[hh][dt] = opaque(tr_hi[dt] + hh * 2 * C::STAGE);
        }
        statp[hh] = opaque(2 * C::TILE + 32 * g + hh * 2 * C::STAGE);
    }
    auto tr16 = [](lds_cptr p) {
        typedef __attribute__((ext_vector_type(4))) short s16x4;
        return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p)));
    };
#define TYR_STG(stg) constexpr int STG = decltype(stg)::value; constexpr int SOFF = (STG & 1) * C::STAGE

    // Row fragments (lane = query row) of sub-tile T of the tile in stage STG
    auto read_rows = [&](auto stg, auto sub, bf16x8 (&qa)[C::KSTEPS], bf16x8 (&da)[C::KSTEPS]) {
        TYR_STG(stg);
        constexpr int T = decltype(sub)::value;
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i) {
            lds_cptr p = rowp[STG >> 1][i] + SOFF + T * 32 * C::ROW;
            qa[i] = *reinterpret_cast<__attribute__((address_space(3))) const bf16x8*>(p);
            da[i] = *reinterpret_cast<__attribute__((address_space(3))) const bf16x8*>(p + C::TILE);
        }
    };
    // S = Q K_w^T and dP = dO V_w^T of one sub-tile from its row fragments
    auto scores = [&](const bf16x8 (&qa)[C::KSTEPS], const bf16x8 (&da)[C::KSTEPS], f32x16& s, f32x16& dp) {
#pragma unroll
        for (int e = 0; e < 16; ++e) { s[e] = 0.0f; dp[e] = 0.0f; }
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i) {
            s = mfma_32x32x16_bf16(qa[i], kf[i], s);
            dp = mfma_32x32x16_bf16(da[i], vf[i], dp);
        }
    };
    // P and dS of a sub-tile as column operands.  Register e <-> query row qs0 + 8(e/4) + 4g + e%4;
    // its (lse2, delta) pair sits at pair index 32T + 8(e/4) + 4g + e%4 of the staged kilobyte.
    // Half sh of the pairs of sub-tile T: registers 8sh .. 8sh+7, i.e. k = e/4 in {2sh, 2sh+1}
    auto read_pairs = [&](auto stg, auto sub, auto half, f32x4 (&st)[4]) {
        TYR_STG(stg);
        constexpr int T = decltype(sub)::value, SH = decltype(half)::value;
        lds_cptr St = statp[STG >> 1] + SOFF + 32 * T * 8;
#pragma unroll
        for (int h = 0; h < 2; ++h) {                    // k = 2 SH + h
            st[2 * h] = *reinterpret_cast<__attribute__((address_space(3))) const f32x4*>(St + 8 * (2 * SH + h) * 8);
            st[2 * h + 1] = *reinterpret_cast<__attribute__((address_space(3))) const f32x4*>(St + 8 * (2 * SH + h) * 8 + 16);
        }
    };
    // P and dS of half sh of a sub-tile (query rows qs0 + 16sh + 8h + 4g + x) as one k-step of column operands
    // `apply` (wave-uniform) says whether any (query, key) pair of the rows at hand is hidden from this
    // wave's keys; the mask instructions are skipped otherwise.
    auto probabilities = [&](auto masked, auto half, const f32x4 (&st)[4], int qs0, const f32x16& s, const f32x16& dp,
                             bf16x8& pf, bf16x8& dsf, bool apply) {
        constexpr bool need_mask = decltype(masked)::value;
        constexpr int sh = decltype(half)::value;
        u32x4 ppk, dpk;
#pragma unroll
        for (int h = 0; h < 2; ++h) {                    // e/4 = 2sh + h
            const f32x4 a = st[2 * h];
            const f32x4 b = st[2 * h + 1];
            const float l2[4] = {a[0], a[2], b[0], b[2]};
            const float dl[4] = {a[1], a[3], b[1], b[3]};
            float p[4], ds[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) p[x] = fast_exp2(fmaf(s[8 * sh + 4 * h + x], scale_log2, -l2[x]));
            if (need_mask && apply) {
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int qrow = qs0 + 8 * (2 * sh + h) + 4 * g + x;
                    const bool hidden = (CAUSAL && kvpos > qrow) ||
                                        (EXT && ((window > 0 && qrow - kvpos >= window) || kvpos >= Nk || key_off));
                    if (hidden) p[x] = 0.0f;
                }
            }
#pragma unroll
            for (int x = 0; x < 4; ++x) ds[x] = p[x] * (dp[8 * sh + 4 * h + x] - dl[x]);
            ppk[2 * h] = pack_bf16(p[0], p[1]);
            ppk[2 * h + 1] = pack_bf16(p[2], p[3]);
            dpk[2 * h] = pack_bf16(ds[0], ds[1]);
            dpk[2 * h + 1] = pack_bf16(ds[2], ds[3]);
        }
        pf = __builtin_bit_cast(bf16x8, ppk);
        dsf = __builtin_bit_cast(bf16x8, dpk);
    };
    // Transposed fragments of k-step c = 2T + sh (query rows 16c + 8h + 4g + [0,4)) of dO and Q
    auto read_transposed = [&](auto stg, int c, bf16x8 (&dot)[C::DT], bf16x8 (&qt)[C::DT]) {
        TYR_STG(stg);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            lds_cptr pl = trlo[STG >> 1][dt] + SOFF + c * 16 * C::ROW;
            lds_cptr ph = trhi[STG >> 1][dt] + SOFF + c * 16 * C::ROW;
            const bf16x4 lo = tr16(pl + C::TILE);
            const bf16x4 hi = tr16(ph + C::TILE);
            dot[dt] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            const bf16x4 ql = tr16(pl);
            const bf16x4 qh = tr16(ph);
            qt[dt] = __builtin_shufflevector(ql, qh, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };

    // With EXT a step applies the mask only where some pair of the 64 query rows it touches (the second
    // half of u, the first half of u+1) is hidden from this wave's keys: a key at or beyond the sequence's
    // length or switched off by the key mask, the causal diagonal, the far edge of the window.
    const bool wave_key_hidden = EXT && __builtin_amdgcn_ballot_w64(kvpos >= Nk || key_off) != 0;
    auto rows_are_masked = [&](int qs0) {
        return wave_key_hidden || (CAUSAL && qs0 < nw0 + 32) || (window > 0 && qs0 + 63 - nw0 >= window);
    };
    bf16x8 rq[C::KSTEPS], rd[C::KSTEPS];              // row fragments of the next sub-tile, read one step ahead
    bf16x8 pf0, dsf0;                                 // P, dS of the first half of the current sub-tile
    f32x4 st1[4];                                     // pairs of its second half
    using Half0 = std::integral_constant<int, 0>;
    using Half1 = std::integral_constant<int, 1>;
    // One step of the software pipeline on sub-tile u = 2t + T, tile t in stage STG (scores in sc / dpc).
    // With one wave per SIMD a vector instruction overlaps with the matrix pipe only where it sits
    // between two MFMAs of the wave's own stream, and the pipe idles through any stretch of vector
    // work that is longer than the MFMA before it.  The step therefore has two phases of 16 MFMAs,
    // each carrying half a sub-tile's exponentials:
    //   A: S, dP of sub-tile u+1 (row fragments already in rq / rd)  beside  P, dS of the second half of u
    //   B: dV, dK of u (both halves)                                  beside  P, dS of the first half of u+1
    // so that P, dS of a sub-tile's first half are always computed one step ahead (pf0 / dsf0).
    // The row fragments of u+2 and the pairs of u+1 are requested a phase before they are used.
    // Past the last sub-tile the "next" reads hit a stage without live data; their results are dropped.
    auto step = [&](auto masked, auto stg, auto sub, int qs0, f32x16& sc, f32x16& dpc, f32x16& sn, f32x16& dpn) {
        constexpr int STG = decltype(stg)::value, T = decltype(sub)::value;
        using Stg1 = std::integral_constant<int, T == 0 ? STG : ((STG + 1) & 3)>;       // stage of u+1
        using Sub1 = std::integral_constant<int, 1 - T>;
        using Stg2 = std::integral_constant<int, (STG + 1) & 3>;                        // stage of u+2
        bf16x8 dot0[C::DT], qt0[C::DT], dot1[C::DT], qt1[C::DT];
        f32x4 st0[4];
        read_transposed(stg, 2 * T, dot0, qt0);
        read_pairs(Stg1{}, Sub1{}, Half0{}, st0);
        read_transposed(stg, 2 * T + 1, dot1, qt1);
        scores(rq, rd, sn, dpn);
        bf16x8 pf1, dsf1;
        const bool apply = decltype(masked)::value && rows_are_masked(qs0);       // rows qs0 .. qs0 + 63
        probabilities(masked, Half1{}, st1, qs0, sc, dpc, pf1, dsf1, apply);
        read_pairs(Stg1{}, Sub1{}, Half1{}, st1);          // ahead of the row fragments: LDS answers in order
        read_rows(Stg2{}, sub, rq, rd);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            dv[dt] = mfma_32x32x16_bf16(dot0[dt], pf0, dv[dt]);
            dk[dt] = mfma_32x32x16_bf16(qt0[dt], dsf0, dk[dt]);
        }
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            dv[dt] = mfma_32x32x16_bf16(dot1[dt], pf1, dv[dt]);
            dk[dt] = mfma_32x32x16_bf16(qt1[dt], dsf1, dk[dt]);
        }
        probabilities(masked, Half0{}, st0, qs0 + 32, sn, dpn, pf0, dsf0, apply);
#ifndef TYR_DKV_NO_SCHED
        // issue order: one MFMA, then its share of the LDS reads and of the vector work
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
        }
#pragma unroll
        for (int i = 0; i < 12; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 1, 0);
        }
#endif
    };
    // What a step expects of the step before it, for the wave's first sub-tile: its scores, P and dS
    // of its first half, the pairs of its second half, and the row fragments of the sub-tile after
    // it.  Without EXT the only partially masked sub-tile of a causal wave is this one (its
    // diagonal): hidden scores become -inf here, which the steps turn into P = 0 and dS = 0 like any
    // other score, so they carry no mask instructions.
    auto first_scores = [&](auto masked, auto stg, auto sub, int qs0, f32x16& sc, f32x16& dpc) {
        constexpr int STG = decltype(stg)::value, T = decltype(sub)::value;
        using Stg1 = std::integral_constant<int, T == 0 ? STG : ((STG + 1) & 3)>;     // stage of u+1
        using Sub1 = std::integral_constant<int, 1 - T>;
        f32x4 st0[4];
        read_rows(stg, sub, rq, rd);
        read_pairs(stg, sub, Half0{}, st0);
        read_pairs(stg, sub, Half1{}, st1);
        scores(rq, rd, sc, dpc);
        if (CAUSAL && !EXT) {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (kvpos > qs0 + 8 * (e >> 2) + 4 * g + (e & 3)) sc[e] = -INFINITY;
        }
        read_rows(Stg1{}, Sub1{}, rq, rd);
        probabilities(masked, Half0{}, st0, qs0, sc, dpc, pf0, dsf0, true);
    };
#undef TYR_STG

#pragma unroll
    for (int i = 0; i < C::KSTEPS; ++i) { pin_registers(kf[i]); pin_registers(vf[i]); }
    for (hq = 0; hq < G; ++hq) {
    issue_tile(0, jq0);
    issue_tile(1, jq0 + 1);
    issue_tile(2, jq0 + 2);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * C::LOADS_PER_TILE) : "memory");
    __syncthreads();

    // Tile t+1 is awaited, and tile t+3 requested into the stage tile t-1 has left, before the
    // first sub-tile of tile t (whose steps already read fragments of tile t+1): four stages.
    auto tile_boundary = [&](int u) {
        if (!(u & 1) && (u >> 1) + 1 < ntile) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(C::LOADS_PER_TILE) : "memory");
            __syncthreads();
            issue_tile(((u >> 1) + 3) & (C::NST - 1), jq0 + (u >> 1) + 3);
        }
    };
    using std::integral_constant;
    using MaskedT = integral_constant<bool, EXT>;
    const int qbase = jq0 * C::BQ;
    // Scores ping-pong between two register sets by the parity of u (no copies).
    f32x16 sA, dpA, sB, dpB;
    int u = 0;
    for (; u < u0 && u < nsub; ++u) tile_boundary(u);           // sub-tiles above the wave's diagonal
    if (u < nsub) {
        // u = u0 < 4: stage u0 / 2, sub-tile u0 % 2; even sub-tiles keep their scores in sA / dpA
        switch (u) {
            case 0:  first_scores(MaskedT{}, integral_constant<int, 0>{}, integral_constant<int, 0>{}, qbase, sA, dpA); break;
            case 1:  first_scores(MaskedT{}, integral_constant<int, 0>{}, integral_constant<int, 1>{}, qbase + 32, sB, dpB); break;
            case 2:  first_scores(MaskedT{}, integral_constant<int, 1>{}, integral_constant<int, 0>{}, qbase + 64, sA, dpA); break;
            default: first_scores(MaskedT{}, integral_constant<int, 1>{}, integral_constant<int, 1>{}, qbase + 96, sB, dpB); break;
        }
    }
    // the pipeline, unrolled over the 8 (stage, sub-tile) combinations; entered at u % 8
#define TYR_STEP(K, CS, CD, NS, ND)                                                                          \
    case K:                                                                                                  \
        if (u >= nsub) goto pipeline_done;                                                                   \
        tile_boundary(u);                                                                                    \
        step(MaskedT{}, integral_constant<int, (K) / 2>{},                                                   \
             integral_constant<int, (K) % 2>{}, qbase + 32 * u, CS, CD, NS, ND);                             \
        ++u;                                                                                                 \
        [[fallthrough]];
    for (;;) {
        switch (u & 7) {
            TYR_STEP(0, sA, dpA, sB, dpB)
            TYR_STEP(1, sB, dpB, sA, dpA)
            TYR_STEP(2, sA, dpA, sB, dpB)
            TYR_STEP(3, sB, dpB, sA, dpA)
            TYR_STEP(4, sA, dpA, sB, dpB)
            TYR_STEP(5, sB, dpB, sA, dpA)
            TYR_STEP(6, sA, dpA, sB, dpB)
            TYR_STEP(7, sB, dpB, sA, dpA)
            default: break;
        }
    }
pipeline_done:
#undef TYR_STEP
    wait_vmcnt0();                                   // drain before the next head reuses the stages
    __syncthreads();
    }

    unsigned char* scratch = lds + w * (32 * (D * 2 + 16));
    store_transposed_bf16<D>(dv, 1.0f, scratch, dV + head_off + (size_t)nw0 * D, N - nw0, lane);
    store_transposed_bf16<D>(dk, scale, scratch, dK + head_off + (size_t)nw0 * D, N - nw0, lane);
}

size_t flash_attn_bwd_workspace_bytes(int B, int H, int N) {
    const size_t npad = (size_t)((N + 127) / 128) * 128;
    return (size_t)B * H * npad * sizeof(float2);
}

int launch_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                          const float* lse, void* dq, void* dk, void* dv, int B, int Hq, int Hkv, int N, int D,
                          int causal, int window, const int* kv_lens, const uint8_t* key_mask, float scale,
                          void* workspace,
                          hipStream_t stream) {
    using namespace fab;
    const int BH = B * Hq, BHkv = B * Hkv, G = Hq / Hkv;
    const int ntq = (N + 127) / 128;
    const int npad = ntq * 128;
    const bool ext = window > 0 || kv_lens != nullptr || key_mask != nullptr;
    const int pair = (causal && window <= 0 && ntq > 1) ? 1 : 0;   // lengths and key masks keep tile 0 starting at key 0
    dim3 grid_q((unsigned)(BH * (pair ? (ntq + 1) / 2 : ntq))), grid_k((unsigned)(BHkv * ntq)), block(THREADS);
    const float scale_log2 = scale * LOG2E;
    auto Qp = static_cast<const uint16_t*>(q);
    auto Kp = static_cast<const uint16_t*>(k);
    auto Vp = static_cast<const uint16_t*>(v);
    auto Op = static_cast<const uint16_t*>(o);
    auto dOp = static_cast<const uint16_t*>(d_o);
    auto st = static_cast<float2*>(workspace);
#define TYR_FAB_LAUNCH(DD, CC, EE)                                                                    \
    do {                                                                                              \
        static const hipError_t a1 = hipFuncSetAttribute(                                             \
            reinterpret_cast<const void*>(&flash_attn_bwd_dq_kernel<DD, CC, EE>),                     \
            hipFuncAttributeMaxDynamicSharedMemorySize, CfgQ<DD>::LDS);                               \
        static const hipError_t a2 = hipFuncSetAttribute(                                             \
            reinterpret_cast<const void*>(&flash_attn_bwd_dkv_kernel<DD, CC, EE>),                    \
            hipFuncAttributeMaxDynamicSharedMemorySize, CfgK<DD>::LDS);                               \
        if (a1 != hipSuccess || a2 != hipSuccess) return -1;                                          \
        hipLaunchKernelGGL((flash_attn_bwd_dq_kernel<DD, CC, EE>), grid_q, block, CfgQ<DD>::LDS, stream, \
                           Qp, Kp, Vp, Op, dOp, lse, static_cast<uint16_t*>(dq), st, BH, N, ntq,      \
                           scale, scale_log2, Hq, G, window, kv_lens, key_mask, pair);                \
        hipLaunchKernelGGL((flash_attn_bwd_dkv_kernel<DD, CC, EE>), grid_k, block, CfgK<DD>::LDS, stream, \
                           Qp, Kp, Vp, dOp, st, static_cast<uint16_t*>(dk),                           \
                           static_cast<uint16_t*>(dv), BHkv, N, ntq, npad, scale, scale_log2, Hq, G,  \
                           window, kv_lens, key_mask);                                                \
    } while (0)
#define TYR_FAB_PICK(DD)                                                                              \
    do {                                                                                              \
        if (ext) { if (causal) TYR_FAB_LAUNCH(DD, true, true); else TYR_FAB_LAUNCH(DD, false, true); }    \
        else     { if (causal) TYR_FAB_LAUNCH(DD, true, false); else TYR_FAB_LAUNCH(DD, false, false); }  \
    } while (0)
    if (D == 128) TYR_FAB_PICK(128); else TYR_FAB_PICK(64);
#undef TYR_FAB_PICK
#undef TYR_FAB_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tyr
