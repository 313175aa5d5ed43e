// Flash-attention forward for gfx950 (bf16 in, f32 softmax, bf16 O + f32 LSE).
//
// Arithmetic contract of the reference (order of operations):
//   Tyr/GPU/Kernels/MhaH100.lean:102-128   S = Q K^T ; S *= scale ; online softmax ; P -> bf16 ;
//                                          O += P V ; O /= l ; LSE = ln l + m ; O -> bf16
//   Tyr/GPU/Codegen/Macros.lean:121-163    m' = max(m,rowmax) ; alpha = exp(m-m') ; O,l *= alpha ;
//                                          P = exp(S-m') ; l += rowsum P(f32)
//   causal semantics: key j visible to query i iff j <= i (cc/src/tyr.cpp:2578-2585, is_causal).
// exp is evaluated as exp2 with log2(e) folded into the scale; the running maximum is advanced
// (and O, l rescaled) only when a row outgrows it by more than a threshold, which is the same
// mathematics with a stale reference point.
//
// Work decomposition.  One workgroup = 4 waves = 128 query rows of one (batch, head); each wave
// owns 32 rows.  Keys/values stream through LDS in tiles of 64 rows, two stages deep, loaded
// directly from global memory into LDS.  The loop is software-pipelined inside each wave: the
// score MFMAs of tile j+1 are issued among the softmax instructions of tile j (so K runs one tile
// ahead of V), which keeps the matrix pipe fed while the vector ALU does the exponentials.
//
// The products are computed transposed so the softmax never leaves the lane:
//   S^T (64 kv x 32 q)  = K_tile (row operand, from LDS)  x  Q^T (column operand, registers)
//   O^T (D x 32 q)     += V_tile^T (row operand, from LDS) x  P^T (column operand, registers)
// With the 32x32 MFMA every lane then holds one query column (l%32) of S^T and O^T: the row
// max/sum are register reductions plus one exchange with lane l^32, the rescale is a per-lane
// scalar, and the exponentials of S^T are already in the register slots the second product
// wants for P^T.  The k index of the second product is a permutation of the kv rows (fixed by
// the accumulator layout of the first).
//
// K and V tiles sit in LDS row-major (one 2D-byte row per kv position, 16-byte chunks XOR-swizzled
// so that neither access pattern has bank conflicts).  K fragments are plain 16-byte reads (lane =
// kv row).  V^T fragments come from ds_read_b64_tr_b16: within each 16-lane block, lane 4q+p
// receives element p of the 8-byte pieces addressed by lanes q, q+4, q+8, q+12 -- so four lanes
// pointing at 4 consecutive d of 4 kv rows hand every lane "its" d for those 4 rows.
#include <limits.h>

#include <atomic>

#include "common.hpp"
#include "launch.hpp"

namespace tyr {

namespace fa {
constexpr int kMaxDevices = 64;
constexpr int BM = 128, BN = 64, THREADS = 256;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float RESCALE_THRESHOLD = 8.0f;

template <int D>
struct Cfg {
    static constexpr int ROW = D * 2;               // bytes per K or V row in LDS
    static constexpr int KCH = D / 8;               // 16-byte chunks per row
    static constexpr int K_TILE = BN * ROW;
    static constexpr int V_TILE = BN * ROW;
    static constexpr int V_BASE = 2 * K_TILE;       // LDS: K stage 0, K stage 1, V stage 0, V stage 1
    static constexpr int LDS = 2 * K_TILE + 2 * V_TILE;
    static constexpr int PER_THREAD = BN * KCH / THREADS;   // 16-byte chunks per thread per tile
    static constexpr int KSTEPS = D / 16;           // MFMA k-steps of Q K^T
    static constexpr int DT = D / 32;               // 32-row tiles of O^T
};

// Swizzles (chunk index within a row -> stored chunk index).
//   K: lanes of one read hold 16 consecutive rows and the same chunk -> spread over all chunks.
//   V: one transposing read touches 4 consecutive rows x 64 bytes per lane-group pair -> move each
//      row of a group of 4 to a different 64-byte quarter... (for D = 64 rows are 128 bytes and the
//      quarter index has one bit less).
template <int D> __device__ __forceinline__ int k_swz(int row, int c) { return c ^ (row & (Cfg<D>::KCH - 1)); }
template <int D> __device__ __forceinline__ int v_swz(int row, int c) { return c ^ (((row & 3) << 2) & (Cfg<D>::KCH - 1)); }
}  // namespace fa

// EXT adds the per-sequence key length (padding mask over the tail) and the sliding window; the
// plain instantiation carries none of their instructions.  G = query heads per kv head.
template <int D, bool CAUSAL, bool EXT>
__global__ __launch_bounds__(fa::THREADS, 2) void flash_attn_fwd_kernel(
    const uint16_t* __restrict__ Q, const uint16_t* __restrict__ Kp, const uint16_t* __restrict__ Vp,
    uint16_t* __restrict__ O, float* __restrict__ LSE, int BH, int N, int ntq, float scale_log2,
    int Hq, int G, int window, const int* __restrict__ kv_lens, const uint8_t* __restrict__ key_mask, int pair,
    int total_ids) {
    using namespace fa;
    using C = Cfg<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int r = lane & 31, g = lane >> 5;

    // workgroup -> (head, query tile).  Heads are dealt to the 8 XCDs so that all query tiles of a
    // head run on one XCD (shared K/V in its L2); within a head the longest (last) causal tiles
    // are issued first.
    // With grouped queries (G > 1) the unit dealt to an XCD is a (batch, kv head) group: its G
    // query heads times ntq tiles share one K/V; the G heads of a tile are adjacent.
    // With `pair` (causal) a workgroup handles query tile ntq-1-tr and then tile tr: every
    // workgroup does the same amount of work and there are half as many of them to start.
    // A launch has either one workgroup per job id, or (persistent launch) two workgroups per CU, of which workgroup p
    // walks the job ids p, p + gridDim.x, ... (the host makes gridDim.x a multiple of 8 then, so with the XCD mapping
    // above all of them belong to its XCD).  The hand-over from a job's last tile to the next job's first one is the
    // hand-over between the two tiles of a pair: the next tile's K(0), K(1) and Q are requested under the end of the
    // current one.
    const int ntr = pair ? (ntq + 1) / 2 : ntq;  // tile ranks per head
    auto decode = [&](int id, int& bh_, int& tr_, int& kvbh_) {
        const int ngroups = BH / G;              // B * Hkv
        if ((ngroups & 7) == 0) {
            const int xcd = id & 7, slot = id >> 3;
            const int per_group = G * ntr;
            kvbh_ = (slot / per_group) * 8 + xcd;
            const int within = slot % per_group;
            tr_ = within / G;
            const int hkv = Hq / G;
            bh_ = (kvbh_ / hkv) * Hq + (kvbh_ % hkv) * G + within % G;
        } else {
            bh_ = id / ntr;
            tr_ = id % ntr;
            kvbh_ = (bh_ / Hq) * (Hq / G) + (bh_ % Hq) / G;
        }
    };
    bf16x8 qf[C::KSTEPS];                        // Q^T fragments: lane holds row qw0+r, columns 16i + 8g + [0,8)
    bool preloaded = false;                      // this tile's K(0), K(1) and Q were requested by the previous one
    for (int id = blockIdx.x; id < total_ids; id += gridDim.x) {
    int bh, tr, kvbh;
    decode(id, bh, tr, kvbh);
    const int npass = (pair && ntq - 1 - tr != tr) ? 2 : 1;
    for (int pass = 0; pass < npass; ++pass) {
    const int qt = CAUSAL ? (pass == 0 ? ntq - 1 - tr : tr) : tr;
    // what this workgroup runs after this tile: the pair's second tile, or the first tile of its next job
    bool has_next = pass + 1 < npass;
    int n_bh = bh, n_kvbh = kvbh, n_qt = tr;
    if (!has_next && id + (int)gridDim.x < total_ids) {
        int n_tr;
        decode(id + (int)gridDim.x, n_bh, n_tr, n_kvbh);
        n_qt = CAUSAL ? ntq - 1 - n_tr : n_tr;
        has_next = true;
    }
    const int q0 = qt * BM;
    const int qw0 = q0 + w * 32;                 // first query row of this wave
    const size_t head_off = (size_t)bh * N * D;
    const size_t kv_head_off = (size_t)kvbh * N * D;
    const uint16_t* Qh = Q + head_off;
    const uint16_t* Kh = Kp + kv_head_off;
    const uint16_t* Vh = Vp + kv_head_off;

    // keys at or beyond Nk are masked (Nk = 0: the sequence has no keys, O = 0 and LSE = -inf); with a window,
    // query i sees keys (i - window, i]
    const int Nk = (EXT && kv_lens != nullptr) ? max(0, min(N, kv_lens[bh / Hq])) : N;
    // per-sequence key mask (nonzero = visible), any pattern
    const uint8_t* km = (EXT && key_mask != nullptr) ? key_mask + (size_t)(bh / Hq) * N : nullptr;
    const int kv_end = CAUSAL ? min(Nk, q0 + BM) : Nk;
    const int nkv_abs = max(1, (kv_end + BN - 1) / BN);   // a sequence without keys still walks one (fully masked) tile
    const int jbase = (EXT && window > 0) ? min(max(0, q0 - window + 1) / BN, nkv_abs - 1) : 0;   // first tile any row sees
    const int nkv = nkv_abs - jbase;             // tiles are numbered from jbase below

    auto load_q = [&](int first_row) {
        const int qrow = min(first_row + r, N - 1);
        const uint16_t* qp = Qh + (size_t)qrow * D + g * 8;
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i)
            qf[i] = __builtin_bit_cast(bf16x8, ld_global_16(qp + i * 16));
    };
    if (!preloaded) load_q(qw0);

    // ---- K/V tile loaders.  Buffer loads: the per-thread byte offset inside a tile is fixed, the
    // tile start is a scalar offset, and rows at or beyond N read as zero (they are masked below).
    const uint32_t head_bytes = (uint32_t)N * D * 2u;
    const u32x4 k_rsrc = make_raw_rsrc(Kh, head_bytes);
    const u32x4 v_rsrc = make_raw_rsrc(Vh, head_bytes);
    const u32x4 nk_rsrc = make_raw_rsrc(Kp + (size_t)n_kvbh * N * D, head_bytes);     // K of the tile after this one
    // Tiles go from global memory straight into LDS (no register staging).  One load instruction
    // of a wave fills 1 KiB of LDS linearly (lane i -> 16 bytes at base + 16 i); the swizzle is
    // applied on the global side: the lane fetches the chunk that belongs at its LDS position.
    constexpr int ROWS_PER_INST = 1024 / C::ROW;
    int gk_voff[C::PER_THREAD], gv_voff[C::PER_THREAD];
#pragma unroll
    for (int m = 0; m < C::PER_THREAD; ++m) {
        const int row = (w * C::PER_THREAD + m) * ROWS_PER_INST + lane / C::KCH;
        const int cpos = lane % C::KCH;                                 // chunk position in LDS
        // (1024 m is taken off: request m carries it as its immediate offset)
        gk_voff[m] = row * C::ROW + k_swz<D>(row, cpos) * 16 - 1024 * m;   // swizzles are involutions
        gv_voff[m] = row * C::ROW + v_swz<D>(row, cpos) * 16 - 1024 * m;
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t wave_dst = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)w * C::PER_THREAD * 1024u);

    auto issue_k = [&](int stage, int j0) {
        const uint32_t dst = wave_dst + (uint32_t)stage * C::K_TILE;
        load_global_to_lds_16xN<C::PER_THREAD>(k_rsrc, dst, gk_voff, j0 * C::ROW);
    };
    auto issue_k_next = [&](int stage, int j0) {
        const uint32_t dst = wave_dst + (uint32_t)stage * C::K_TILE;
        load_global_to_lds_16xN<C::PER_THREAD>(nk_rsrc, dst, gk_voff, j0 * C::ROW);
    };
    auto issue_v = [&](int stage, int j0) {
        const uint32_t dst = wave_dst + C::V_BASE + (uint32_t)stage * C::V_TILE;
        load_global_to_lds_16xN<C::PER_THREAD>(v_rsrc, dst, gv_voff, j0 * C::ROW);
    };

    f32x16 oacc[C::DT];
#pragma unroll
    for (int i = 0; i < C::DT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[i][e] = 0.0f;
    // running row maximum, in log2 units (score * scale * log2 e).  With a window a row's first
    // tiles can be wholly masked; a finite start keeps (-inf) - m2 from becoming NaN there.
    float m2 = EXT ? -1.0e30f : -INFINITY;
    float lsum = 0.0f;         // this lane's share of the running row sum

    // K fragment (sub-tile T, k-step i): row 32T + r, chunk 2i + g.
    int k_roff[C::KSTEPS];
#pragma unroll
    for (int i = 0; i < C::KSTEPS; ++i) k_roff[i] = r * C::ROW + k_swz<D>(r, 2 * i + g) * 16;
    // V^T fragment (d tile dt; rows 32T + 16s + 8h + 4g + [0,4)): as a source lane of the transposing
    // read this lane points at row 4g + (lane%16)/4 of that group, 8 bytes at d = 32dt + 16(b&1) + 4(lane%4).
    int v_roff[C::DT];
    {
        const int i16 = lane & 15, b16 = lane >> 4;
        const int row = 4 * (b16 >> 1) + (i16 >> 2);
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
            const int dcol = 32 * dt + 16 * (b16 & 1) + 4 * (i16 & 3);
            v_roff[dt] = C::V_BASE + row * C::ROW + v_swz<D>(row, dcol >> 3) * 16 + (dcol & 7) * 2;
        }
    }
    const int qpos = qw0 + r;
    // The second tile of a pair starts under the end of the first: its K(0), K(1) are requested
    // in the first tile's last two steps (stage parity needs an even tile count), its Q rows
    // before the first tile's output is written.
    const bool overlap_next = has_next && (nkv & 1) == 0 && !(EXT && window > 0);
    // number of kv tiles that intersect this wave's visible region
    const int nkv_w = CAUSAL ? min(nkv, (qw0 + 31) / BN + 1 - jbase) : nkv;

    constexpr int NG = C::KSTEPS / 2;            // S^T is built in NG groups of (2 k-steps x 2 sub-tiles)
    auto read_k_group = [&](const unsigned char* Kt, int grp, bf16x8 (&dst)[4]) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            dst[u] = *reinterpret_cast<const bf16x8*>(Kt + k_roff[2 * grp + (u >> 1)] + (u & 1) * 32 * C::ROW);
    };
    auto mfma_k_group = [&](f32x16 (&sacc)[2], int grp, const bf16x8 (&kf)[4]) {
#pragma unroll
        for (int u = 0; u < 4; ++u) sacc[u & 1] = mfma_32x32x16_bf16(kf[u], qf[2 * grp + (u >> 1)], sacc[u & 1]);
    };
    auto zero_s = [&](f32x16 (&sacc)[2]) {
#pragma unroll
        for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[T][e] = 0.0f;
    };

    // ---- prologue: K(0), V(0), K(1) in flight; S(0) computed on its own
    if (!preloaded) {
        issue_k(0, jbase * BN);
        issue_v(0, jbase * BN);
        if (nkv > 1) issue_k(1, (jbase + 1) * BN);
    } else {
        issue_v(0, 0);                           // K(0), K(1) and Q were requested by the first tile
    }
#pragma unroll
    for (int i = 0; i < C::KSTEPS; ++i) pin_registers(qf[i]);
    wait_vmcnt0();
    __syncthreads();

    f32x16 sA[2], sB[2];
    zero_s(sA);
    {
        bf16x8 kf[2][4];
        read_k_group(lds, 0, kf[0]);
#pragma unroll
        for (int grp = 0; grp < NG; ++grp) {
            if (grp + 1 < NG) read_k_group(lds, grp + 1, kf[(grp + 1) & 1]);
            mfma_k_group(sA, grp, kf[grp & 1]);
        }
    }
    // Every wave has read K(0) before any wave's first tile step requests K(2) into the same stage.  (From the
    // second step on the barrier at the end of a step separates the reads of a stage from its next request; the
    // prologue has none of its own, and a request that is served by the L2 can land within a few hundred
    // nanoseconds -- less than a wave can lag behind another that shares its SIMD with a second workgroup.)
    __syncthreads();

    // One kv tile: softmax and P V of tile j (scores in `cur`), overlapped with the score MFMAs of
    // tile j+1 (into `nxt`).  K runs one tile ahead of V in LDS: at entry K(j+1) and V(j) are
    // resident; K(j+2) and V(j+1) are requested here and awaited at the end.
    auto tile_step = [&](f32x16 (&cur)[2], f32x16 (&nxt)[2], int j) {
        const int j0 = (jbase + j) * BN;
        // The two requests are issued apart (K here, V after the row-max reduction) so the waves of
        // a CU do not all queue on the texture path at once.
        // In the last two steps of the first tile of a pair the freed K stages take K(0) and K(1) of
        // the second tile (a full one, >= 2 kv tiles, starting from key 0).
        if (j + 2 < nkv) issue_k(j & 1, j0 + 2 * BN);
        else if (overlap_next) issue_k_next(j & 1, (j + 2 - nkv) * BN);
        if (j >= nkv_w && j + 1 < nkv) issue_v((j + 1) & 1, j0 + BN);

        if (j < nkv_w) {
            const unsigned char* Kt = lds + ((j + 1) & 1) * C::K_TILE;     // K(j+1) (stale on the last tile: unused)
            const unsigned char* Vt = lds + (j & 1) * C::V_TILE;           // V(j), v_roff carries V_BASE

            // ---- mask (diagonal tiles, ragged tail) -- register e of sub-tile T is kv row
            //      j0 + 32T + 8(e/4) + 4g + e%4
            // The tile's 64 key-mask bytes are the same for every lane: lane l reads the byte of kv row
            // j0 + l and a ballot makes them one 64-bit word (bit r set: row j0 + r is hidden).  A tile
            // without hidden rows skips the masking.  (Rows at or beyond N are hidden by `lim` already.)
            uint64_t tile_hidden = 0;
            if (EXT && km != nullptr) tile_hidden = __builtin_amdgcn_ballot_w64(km[min(j0 + lane, N - 1)] == 0);
            const bool need_mask = (CAUSAL && (j0 + BN - 1 > qw0)) || (j0 + BN > Nk) ||
                                   (EXT && window > 0 && j0 < qw0 + 32 - window) || (EXT && tile_hidden != 0);
            if (need_mask) {
                const int lim = CAUSAL ? min(qpos, Nk - 1) : Nk - 1;   // largest visible kv row
                const int low = (EXT && window > 0) ? qpos - window + 1 : INT_MIN;   // smallest visible kv row
                const int base = j0 + 4 * g;
                const uint64_t hidden = tile_hidden >> (4 * g);      // shifted to this lane's rows
#pragma unroll
                for (int T = 0; T < 2; ++T)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int kv = base + 32 * T + 8 * (e >> 2) + (e & 3);
                        const bool off = kv > lim || (EXT && kv < low) ||
                                         ((hidden >> (32 * T + 8 * (e >> 2) + (e & 3))) & 1u);
                        cur[T][e] = off ? -INFINITY : cur[T][e];
                    }
            }

            // ---- next tile's scores, first group, under the row-max reduction of this tile
            bf16x8 kf[2][4];
            zero_s(nxt);
            read_k_group(Kt, 0, kf[0]);
            read_k_group(Kt, 1, kf[1]);

            // online softmax on this lane's query column.  The reference maximum m2 is only
            // advanced (and O, l rescaled) when some row of the wave outgrew it by more than
            // RESCALE_THRESHOLD (in log2 units); otherwise exp2(s - m2) <= 2^threshold, which f32
            // sums and bf16 P hold without loss.
            float mx = cur[0][0];
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, cur[T][e]);
            mfma_k_group(nxt, 0, kf[0]);
            mx = max_xor32(mx) * scale_log2;
            if (__builtin_amdgcn_ballot_w64(mx > m2 + RESCALE_THRESHOLD) != 0) {
                const float m2new = fmaxf(m2, mx);
                const float alpha = fast_exp2(m2 - m2new);
#pragma unroll
                for (int i = 0; i < C::DT; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) oacc[i][e] *= alpha;
                lsum *= alpha;
                m2 = m2new;
            }

            if (j + 1 < nkv) issue_v((j + 1) & 1, j0 + BN);

            // ---- exponentials of this tile under the remaining score MFMAs of the next
            float psum = 0.0f;
            bf16x8 pf[2][2];
            bf16x8 vf[2][C::DT];
            auto read_v_group = [&](int c, bf16x8 (&dst)[C::DT]) {
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt) {
                    const unsigned char* p = Vt + v_roff[dt] + c * 16 * C::ROW;   // rows 16c + ...
                    const bf16x4 lo = ds_read_tr16(p);
                    const bf16x4 hi = ds_read_tr16(p + 8 * C::ROW);
                    dst[dt] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
            };
#pragma unroll
            for (int c = 0; c < 4; ++c) {                 // c = 2T + s : 8 scores each
                const int T = c >> 1, sh = c & 1;
                if (c + 1 < NG) {
                    if (c + 2 < NG) read_k_group(Kt, c + 2, kf[c & 1]);
                    mfma_k_group(nxt, c + 1, kf[(c + 1) & 1]);
                }
                if (c == 3) read_v_group(0, vf[0]);       // first V^T fragments arrive under the last exponentials
                u32x4 pk;
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const float p0 = fast_exp2(fmaf(cur[T][8 * sh + 2 * jj], scale_log2, -m2));
                    const float p1 = fast_exp2(fmaf(cur[T][8 * sh + 2 * jj + 1], scale_log2, -m2));
                    psum += p0 + p1;
                    pk[jj] = pack_bf16(p0, p1);
                }
                pf[T][sh] = __builtin_bit_cast(bf16x8, pk);
            }
            lsum += psum;

            // ---- O^T += V^T P^T; fragment reads run one group ahead.  Group c = (T, s).
            {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (c + 1 < 4) read_v_group(c + 1, vf[(c + 1) & 1]);
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
                        oacc[dt] = mfma_32x32x16_bf16(vf[c & 1][dt], pf[c >> 1][c & 1], oacc[dt]);
                }
            }
        }

        wait_vmcnt0();
        __syncthreads();
    };

    for (int j = 0; j < nkv; j += 2) {
        tile_step(sA, sB, j);
        if (j + 1 < nkv) tile_step(sB, sA, j + 1);
    }

    // ---- finalize: O /= l, LSE = ln l + m.  The wave's 32 x D block of O goes through a private LDS
    // scratch in the V stages (dead after the last barrier; the K stages may already be filling for
    // the second tile of a pair) so that global stores are 16 bytes per lane along rows.  Rows are
    // unpadded; 16-byte chunks are XOR-swizzled by row.
    if (overlap_next) {
        const int qrow = min(n_qt * BM + w * 32 + r, N - 1);
        const uint16_t* qp = Q + (size_t)n_bh * N * D + (size_t)qrow * D + g * 8;
#pragma unroll
        for (int i = 0; i < C::KSTEPS; ++i) qf[i] = __builtin_bit_cast(bf16x8, ld_global_16(qp + i * 16));
    }
    const float ltot = sum_xor32(lsum);
    const float inv = (!EXT || ltot > 0.0f) ? 1.0f / ltot : 0.0f;    // EXT: a row that saw no key gives 0
    {
        constexpr int SROW = D * 2;
        constexpr int CH = D / 8;                   // 16-byte chunks per row
        auto s_swz = [](int row) { return (D == 128 ? row : (row >> 1)) & (CH - 1); };
        unsigned char* scratch = lds + C::V_BASE + w * (32 * SROW);
        int wr_swz = s_swz(r) * 16;
        asm volatile("" : "+v"(wr_swz));            // keeps the 16 swizzled addresses out of the main loop's registers
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                u32x2 v;
                v.x = pack_bf16(oacc[dt][4 * q4 + 0] * inv, oacc[dt][4 * q4 + 1] * inv);
                v.y = pack_bf16(oacc[dt][4 * q4 + 2] * inv, oacc[dt][4 * q4 + 3] * inv);
                *reinterpret_cast<u32x2*>(scratch + r * SROW + (((dt * 4 + q4) * 16) ^ wr_swz) + g * 8) = v;
            }
        }
        constexpr int RPI = 64 / CH;                // rows per store instruction
#pragma unroll
        for (int k = 0; k < 32 / RPI; ++k) {
            const int row = lane / CH + RPI * k;
            const u32x4 v = *reinterpret_cast<const u32x4*>(scratch + row * SROW + ((lane % CH) ^ s_swz(row)) * 16);
            if (qw0 + row < N) st_global_16(O + head_off + (size_t)(qw0 + row) * D + (lane % CH) * 8, v);
        }
    }
    if (qpos < N && LSE != nullptr && g == 0) LSE[(size_t)bh * N + qpos] = logf(ltot) + m2 * LN2;
    __syncthreads();                             // the scratch is read; the stages may be refilled
    preloaded = overlap_next;
    }
    }
}

int launch_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                          int Hq, int Hkv, int N, int D, int causal, int window, const int* kv_lens,
                          const uint8_t* key_mask,
                          float scale, hipStream_t stream) {
    using namespace fa;
    const int BH = B * Hq;
    const int G = Hq / Hkv;
    const int ntq = (N + BM - 1) / BM;
    const bool ext = window > 0 || kv_lens != nullptr || key_mask != nullptr;
    const int pair = (causal && window <= 0 && ntq > 1) ? 1 : 0;   // lengths and key masks keep tile 0 starting at key 0
    const int total_ids = BH * (pair ? (ntq + 1) / 2 : ntq);
    // One workgroup per job id, or persistent workgroups: two per CU (what registers and 64 KB of LDS at D = 128 allow),
    // rounded down to a multiple of 8 so that a workgroup's job ids stay on one XCD, and never fewer than 8.
    unsigned nwg = (unsigned)total_ids;
    if (flash_attn_fwd_persistent()) {
        static std::atomic<int> resident_of[kMaxDevices];       // per device, 0 = not asked yet
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
        int resident = resident_of[dev].load(std::memory_order_relaxed);
        if (resident == 0) {
            int cus = 0;
            if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
            resident = 2 * cus / 8 * 8;
            if (resident < 8) resident = 8;
            resident_of[dev].store(resident, std::memory_order_relaxed);
        }
        if (total_ids > resident) nwg = (unsigned)resident;
    }
    dim3 grid(nwg), block(THREADS);
    const float scale_log2 = scale * LOG2E;
    auto Qp = static_cast<const uint16_t*>(q);
    auto Kp = static_cast<const uint16_t*>(k);
    auto Vp = static_cast<const uint16_t*>(v);
    auto Op = static_cast<uint16_t*>(o);
#define TYR_FA_LAUNCH(DD, CC, EE)                                                                \
    do {                                                                                         \
        static const hipError_t attr = hipFuncSetAttribute(                                      \
            reinterpret_cast<const void*>(&flash_attn_fwd_kernel<DD, CC, EE>),                   \
            hipFuncAttributeMaxDynamicSharedMemorySize, Cfg<DD>::LDS);                           \
        if (attr != hipSuccess) return -1;                                                       \
        hipLaunchKernelGGL((flash_attn_fwd_kernel<DD, CC, EE>), grid, block, Cfg<DD>::LDS, stream, \
                           Qp, Kp, Vp, Op, lse, BH, N, ntq, scale_log2, Hq, G, window, kv_lens, key_mask, pair, total_ids); \
    } while (0)
#define TYR_FA_PICK(DD)                                                                          \
    do {                                                                                         \
        if (ext) { if (causal) TYR_FA_LAUNCH(DD, true, true); else TYR_FA_LAUNCH(DD, false, true); }   \
        else     { if (causal) TYR_FA_LAUNCH(DD, true, false); else TYR_FA_LAUNCH(DD, false, false); } \
    } while (0)
    if (D == 128) TYR_FA_PICK(128); else TYR_FA_PICK(64);
#undef TYR_FA_PICK
#undef TYR_FA_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tyr
