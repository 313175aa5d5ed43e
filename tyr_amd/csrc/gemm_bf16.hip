// bf16 GEMM for gfx950: C[M,N] = A[M,K] * B  (B is [K,N], or [N,K] when TRANS_B), f32
// accumulation on the 32x32x16 bf16 MFMA, bf16 output.
//
// Arithmetic contract of the reference: Tyr/GPU/Kernels/GemmCommon.lean:22-69
// (tiledAccumulator + storeConvertedTile: f32 accumulate, convert once at the end),
// Tyr/GPU/Kernels/Examples.lean:23-65 (B as K x N), cc/src/tyr.cpp:1602-1607 (torch::mm).
//
// Design (one workgroup = 256 threads = 4 waves, 1 workgroup per CU):
//   * 256x256 output tile, K consumed in slices of 64.  Each wave owns a 128x128 quadrant:
//     4x4 MFMA tiles of 32x32, 256 accumulator registers per lane.
//   * Both operands are staged in LDS as k-contiguous rows (128 B + 16 B pad, which makes the
//     16-byte MFMA operand reads of 16 consecutive rows hit 64 distinct banks).  When B is
//     [K,N] the loader transposes 8x8 blocks in registers on the way to LDS, so the inner loop
//     is identical for both layouts.
//   * Two LDS stages; the next K slice is fetched into registers while the current one is
//     multiplied, then written to the other stage: one barrier per slice.
//   * The MFMA is issued with the B fragment as its row operand, so every lane ends up with
//     4 consecutive n for one m and stores 8-byte pieces of a C row.
#include "common.hpp"
#include "launch.hpp"

namespace tyr {

namespace gemm {
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int ROW_BYTES = BK * 2 + 16;           // 144
constexpr int TILE_BYTES = BM * ROW_BYTES;       // 36864 per operand per stage
constexpr int LDS_BYTES = 4 * TILE_BYTES;        // A0 B0 A1 B1 = 147456
constexpr int THREADS = 256;
constexpr int GROUP_M = 4;
}  // namespace gemm

template <bool TRANS_B, bool EDGE>
__global__ __launch_bounds__(gemm::THREADS) void gemm_bf16_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, int tiles_m, int tiles_n, long stride_a, long stride_b, long stride_c) {
    using namespace gemm;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    // batch entry blockIdx.y (element strides; stride_b = 0 broadcasts one B)
    A += (size_t)blockIdx.y * stride_a;
    B += (size_t)blockIdx.y * stride_b;
    C += (size_t)blockIdx.y * stride_c;

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int wm = w >> 1, wn = w & 1;

    // workgroup -> output tile: XCD-contiguous logical order, then grouped (GROUP_M tile rows
    // are walked column by column) so that one XCD's 32 tiles share few A and B panels.
    const uint32_t nblk = (uint32_t)tiles_m * (uint32_t)tiles_n;
    const uint32_t pid = xcd_remap(blockIdx.x, nblk);
    const uint32_t per_group = GROUP_M * (uint32_t)tiles_n;
    const uint32_t grp = pid / per_group;
    const uint32_t first_m = grp * GROUP_M;
    const uint32_t gsz = min((uint32_t)tiles_m - first_m, (uint32_t)GROUP_M);
    const int tm = (int)(first_m + (pid % per_group) % gsz);
    const int tn = (int)((pid % per_group) / gsz);
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- loader coordinates
    // A (and B when TRANS_B): 8 chunks of 16 B per thread; chunk c -> row c/8, k-chunk c%8.
    // B when !TRANS_B: one 8(k) x 8(n) block per thread: kb = t%8, nb = t/8.
    u32x4 ra[8], rb[8];

    auto load_slice = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = t + THREADS * i;
            const int row = c >> 3, kc = c & 7;
            const int gm = m0 + row, gk = k0 + kc * 8;
            if (!EDGE || (gm < M && gk < K))
                ra[i] = ld_global_16(A + (size_t)gm * K + gk);
            else
                ra[i] = u32x4{0, 0, 0, 0};
        }
        if (TRANS_B) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = t + THREADS * i;
                const int row = c >> 3, kc = c & 7;
                const int gn = n0 + row, gk = k0 + kc * 8;
                if (!EDGE || (gn < N && gk < K))
                    rb[i] = ld_global_16(B + (size_t)gn * K + gk);
                else
                    rb[i] = u32x4{0, 0, 0, 0};
            }
        } else {
            const int kb = t & 7, nb = t >> 3;
            const int gn = n0 + nb * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int gk = k0 + kb * 8 + i;
                if (!EDGE || (gk < K && gn < N))
                    rb[i] = ld_global_16(B + (size_t)gk * N + gn);
                else
                    rb[i] = u32x4{0, 0, 0, 0};
            }
        }
    };

    auto store_slice = [&](int stage) {
        unsigned char* As = lds + stage * 2 * TILE_BYTES;
        unsigned char* Bs = As + TILE_BYTES;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = t + THREADS * i;
            *reinterpret_cast<u32x4*>(As + (c >> 3) * ROW_BYTES + (c & 7) * 16) = ra[i];
        }
        if (TRANS_B) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int c = t + THREADS * i;
                *reinterpret_cast<u32x4*>(Bs + (c >> 3) * ROW_BYTES + (c & 7) * 16) = rb[i];
            }
        } else {
            const int kb = t & 7, nb = t >> 3;
            u32x4 tr[8];
            transpose8x8_b16(rb, tr);
#pragma unroll
            for (int j = 0; j < 8; ++j)
                *reinterpret_cast<u32x4*>(Bs + (nb * 8 + j) * ROW_BYTES + kb * 16) = tr[j];
        }
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const int KT = (K + BK - 1) / BK;
    load_slice(0);
    store_slice(0);
    __syncthreads();

    const int a_off = (wm * 128 + r) * ROW_BYTES + g * 16;
    const int b_off = (wn * 128 + r) * ROW_BYTES + g * 16;

    for (int kt = 0; kt < KT; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < KT) load_slice((kt + 1) * BK);

        const unsigned char* As = lds + stage * 2 * TILE_BYTES + a_off;
        const unsigned char* Bs = lds + stage * 2 * TILE_BYTES + TILE_BYTES + b_off;
#pragma unroll
        for (int s = 0; s < BK / 16; ++s) {
            bf16x8 af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                af[i] = *reinterpret_cast<const bf16x8*>(As + i * 32 * ROW_BYTES + s * 32);
                bf[i] = *reinterpret_cast<const bf16x8*>(Bs + i * 32 * ROW_BYTES + s * 32);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mfma_32x32x16_bf16(bf[j], af[i], acc[i][j]);
        }

        if (kt + 1 < KT) store_slice(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds m = ..+r and, per register quad q4, n = ..+8*q4+4*g+[0,4)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + wm * 128 + i * 32 + r;
        if (EDGE && gm >= M) continue;
        uint16_t* crow = C + (size_t)gm * N;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int gn = n0 + wn * 128 + j * 32 + q4 * 8 + g * 4;
                if (EDGE && gn >= N) continue;
                u32x2 v;
                v.x = pack_bf16(acc[i][j][q4 * 4 + 0], acc[i][j][q4 * 4 + 1]);
                v.y = pack_bf16(acc[i][j][q4 * 4 + 2], acc[i][j][q4 * 4 + 3]);
                st_global_8(crow + gn, v);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Fast path for K % 8 == 0 (any M; N % 8 == 0; a last slice shorter than 64 is zero-filled).
//
// Same 256x256x64 decomposition, but the slices travel from global memory straight into LDS
// (no register staging, no LDS stores from the ALU), rows are unpadded with XOR-swizzled 16-byte
// chunks, and when B is [K,N] it stays row-major in LDS: its MFMA fragments (8 consecutive k for
// one n) are gathered by the transposing LDS read.  Fragments for k-step s+1 are requested before
// the 16 MFMAs of k-step s are issued.
namespace gemm2 {
constexpr int BM = 256, BN = 256, BK = 64, THREADS = 512;
constexpr int A_TILE = BM * BK * 2;                  // 32 KiB: [256 m][8 chunks]
constexpr int B_TILE = BN * BK * 2;                  // 32 KiB: [64 k][32 chunks] or [256 n][8 chunks]
constexpr int STAGE = A_TILE + B_TILE;
constexpr int LDS_BYTES = 2 * STAGE;                 // 128 KiB
constexpr int GROUP_M = 4;
}  // namespace gemm2

template <bool TRANS_B, bool K_TAIL>
__global__ __launch_bounds__(gemm2::THREADS, 1) void gemm_bf16_fast_kernel(
    const uint16_t* __restrict__ A, const uint16_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, int tiles_m, int tiles_n, long stride_a, long stride_b, long stride_c) {
    using namespace gemm2;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    A += (size_t)blockIdx.y * stride_a;
    B += (size_t)blockIdx.y * stride_b;
    C += (size_t)blockIdx.y * stride_c;

    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, g = lane >> 5;
    const int wm = w >> 2, wn = w & 3;                 // eight waves: wave (wm, wn) owns 128 rows x 64 columns

    const uint32_t nblk = (uint32_t)tiles_m * (uint32_t)tiles_n;
    const uint32_t pid = xcd_remap(blockIdx.x, nblk);
    const uint32_t per_group = GROUP_M * (uint32_t)tiles_n;
    const uint32_t grp = pid / per_group;
    const uint32_t first_m = grp * GROUP_M;
    const uint32_t gsz = min((uint32_t)tiles_m - first_m, (uint32_t)GROUP_M);
    const int tm = (int)(first_m + (pid % per_group) % gsz);
    const int tn = (int)((pid % per_group) / gsz);
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> LDS requests.  Each wave owns an eighth of each tile: 4 instructions of 1 KiB.
    // A (and B when TRANS_B): 8 rows of 128 B per instruction; chunk c of row m is stored at
    // position c ^ ((m >> 1) & 7), so 16 consecutive rows put one logical chunk on all 64 banks.  B when !TRANS_B: 2 rows of 512 B per instruction; chunk c of row k is
    // stored at position c ^ ((k & 3) << 2).
    // (a descriptor spans the tile's rows only and stays below 2 GiB, so that the offset 2^31 given to
    //  the chunks past K of a ragged last slice is out of range whatever is added to it)
    const u32x4 a_rsrc = make_raw_rsrc(A + (size_t)m0 * K, (uint32_t)((size_t)min(M - m0, BM) * K * 2));
    const u32x4 b_rsrc = TRANS_B
        ? make_raw_rsrc(B + (size_t)n0 * K, (uint32_t)((size_t)min(N - n0, BN) * K * 2))
        // (descriptor shifted down by 3072 bytes: with few columns a row is shorter than the kilobytes taken
        //  off the per-lane offsets below, and those must not go negative)
        : make_raw_rsrc(B + n0 - 1536, (uint32_t)min(((size_t)K * N - n0) * 2 + 3072, (size_t)0xffffffffu));
    int a_voff[4], b_voff[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const int row = (w * 4 + m) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        // (1024 m is taken off: the request carries it as its immediate offset, see issue)
        a_voff[m] = row * K * 2 + c * 16 - 1024 * m;
        if (TRANS_B) {
            b_voff[m] = row * K * 2 + c * 16 - 1024 * m;
        } else {
            const int krow = (w * 4 + m) * 2 + (lane >> 5);
            const int cb = (lane & 31) ^ ((krow & 3) << 2);
            b_voff[m] = krow * N * 2 + cb * 16 - 1024 * m + 3072;
        }
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t wave_dst = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)w * 4096u);
    // the wave's requests for slice kt into stage st: part 0 the A tile, part 1 the B tile, four instructions
    // behind one M0 write each (the immediate offset steps the LDS destination by a kilobyte)
    const int KT = (K + BK - 1) / BK;
    auto issue = [&](int st, int kt, int part) {
        const int a_soff = kt * BK * 2;
        const int b_soff = TRANS_B ? kt * BK * 2 : kt * BK * N * 2;
        const uint32_t dst = wave_dst + (uint32_t)st * STAGE;
        int av[4] = {a_voff[0], a_voff[1], a_voff[2], a_voff[3]};
        int bv[4] = {b_voff[0], b_voff[1], b_voff[2], b_voff[3]};
        if (K_TAIL && kt == KT - 1) {
            // ragged last slice (K % 8 == 0): the 16-byte chunks of a row at k >= K belong to the next
            // row and must read as zeros; rows k >= K of a [K,N] B are past its descriptor already
            const int chunks = (K - kt * BK) >> 3;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = (w * 4 + i) * 8 + (lane >> 3);
                const int c = (lane & 7) ^ ((row >> 1) & 7);
                if (c >= chunks) {
                    av[i] = (int)0x80000000u;
                    if (TRANS_B) bv[i] = (int)0x80000000u;
                }
            }
        }
        if (part == 0) load_global_to_lds_16xN<4>(a_rsrc, dst, av, a_soff);
        else           load_global_to_lds_16xN<4>(b_rsrc, dst + A_TILE, bv, b_soff);
    };

    // ---- fragment addresses
    // A fragment (m tile i, k-step s): row wm*128 + 32i + r, chunk (2s + g) ^ ((r >> 1) & 7).
    int a_roff[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) a_roff[s] = (wm * 128 + r) * 128 + (((2 * s + g) ^ ((r >> 1) & 7)) * 16);
    // B fragment, TRANS_B: like A with n rows.  Otherwise (row-major [k][n]) via the transposing
    // read: as a source lane this lane points at k row 8(b/2) + 4h + j (j = (lane%16)/4) of the
    // k-step, 8 bytes at n = wn*64 + 32jt + 16(b&1) + 4(lane%4); jt enters through the swizzle.
    int b_roff[4];
    if (TRANS_B) {
#pragma unroll
        for (int s = 0; s < 4; ++s) b_roff[s] = A_TILE + (wn * 64 + r) * 128 + (((2 * s + g) ^ ((r >> 1) & 7)) * 16);
    } else {
        const int i16 = lane & 15, b16 = lane >> 4;
        const int js = i16 >> 2, qs = i16 & 3;
        const int krow = 8 * (b16 >> 1) + js;
#pragma unroll
        for (int jt = 0; jt < 2; ++jt) {
            const int c = wn * 8 + 4 * jt + 2 * (b16 & 1) + (qs >> 1);
            b_roff[jt] = A_TILE + krow * 512 + ((c ^ (js << 2)) * 16) + (qs & 1) * 8;
        }
        b_roff[2] = b_roff[3] = 0;
    }

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    // fragments of k-step s: A of m tile i, B of n tile j
    auto read_a = [&](const unsigned char* St, int s, int i, bf16x8& fa) {
        fa = *reinterpret_cast<const bf16x8*>(St + a_roff[s] + i * 32 * 128);
    };
    auto read_b = [&](const unsigned char* St, int s, int j, bf16x8& fb) {
        if (TRANS_B) {
            fb = *reinterpret_cast<const bf16x8*>(St + b_roff[s] + j * 32 * 128);
        } else {
            const unsigned char* p = St + b_roff[j] + s * 16 * 512;
            const bf16x4 lo = ds_read_tr16(p);
            const bf16x4 hi = ds_read_tr16(p + 4 * 512);
            fb = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };

    issue(0, 0, 0);
    issue(0, 0, 1);
    wait_vmcnt0();
    __syncthreads();

    // Steady state per slice: the next slice is requested during k-steps 0 and 1; the fragments of
    // k-step s+1 are read during the MFMAs of k-step s; in the middle of the last k-step the workgroup
    // waits for the requests, synchronises and reads the first fragments of the next slice.  Two waves
    // share a SIMD, so what one waits for is covered by the other's MFMAs; requests and fragment reads
    // are still dealt out between the MFMA rows (2 MFMAs, 64 cycles each) and the scheduling barriers
    // keep that order.
    // (Past the last slice the requests and reads touch the idle stage / stale data and are never used.)
    bf16x8 af[2][4], bf[2][2];
#pragma unroll
    for (int i = 0; i < 4; ++i) read_a(lds, 0, i, af[0][i]);
#pragma unroll
    for (int j = 0; j < 2; ++j) read_b(lds, 0, j, bf[0][j]);
#define TYR_FENCE __builtin_amdgcn_sched_barrier(0)
    for (int kt = 0; kt < KT; ++kt) {
        const int st = kt & 1;
        const unsigned char* St = lds + st * STAGE;
        const unsigned char* Sn = lds + (st ^ 1) * STAGE;
        auto row = [&](int b, int i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x16_bf16(bf[b][j], af[b][i], acc[i][j]);
        };
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int cb = s & 1, nb = cb ^ 1;
            if (s < 3) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (s < 2 && i == 0) issue(st ^ 1, kt + 1, s);
                    read_a(St, s + 1, i, af[nb][i]);
                    if (i < 2) read_b(St, s + 1, i, bf[nb][i]);
                    TYR_FENCE; row(cb, i); TYR_FENCE;
                }
            } else {
                row(cb, 0); TYR_FENCE;
                row(cb, 1); TYR_FENCE;
                wait_vmcnt0();
                __syncthreads();
                read_a(Sn, 0, 0, af[nb][0]);
                read_b(Sn, 0, 0, bf[nb][0]);
                read_b(Sn, 0, 1, bf[nb][1]);
                TYR_FENCE; row(cb, 2); TYR_FENCE;
                read_a(Sn, 0, 1, af[nb][1]);
                read_a(Sn, 0, 2, af[nb][2]);
                read_a(Sn, 0, 3, af[nb][3]);
                TYR_FENCE; row(cb, 3); TYR_FENCE;
            }
        }
    }
#undef TYR_FENCE

    // ---- epilogue (all requests have landed and every wave is past its last fragment read)
    store_quadrant_bf16<2>(acc, 1.0f, lds + w * kEpilogueScratchBytes,
                           C + (size_t)(m0 + wm * 128) * N + n0 + wn * 64, N, lane,
                           M - (m0 + wm * 128), N - (n0 + wn * 64));
}

int launch_gemm_bf16(const void* a, const void* b, void* c, int M, int N, int K, int trans_b,
                     int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, hipStream_t stream) {
    using namespace gemm;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const bool edge = (M % BM) || (N % BN) || (K % BK);
    dim3 grid((unsigned)(tiles_m * tiles_n), (unsigned)batch), block(THREADS);
    auto A = static_cast<const uint16_t*>(a);
    auto Bp = static_cast<const uint16_t*>(b);
    auto Cp = static_cast<uint16_t*>(c);
    // 32-bit buffer offsets: one 256-row panel of A (and of B^T), or all of B, must stay below 4 GiB
    // The fast kernel needs rows of whole 16-byte chunks; ragged M, N and K are handled by the zero
    // fill of the buffer loads (rows past the end, chunks past K) and by the guarded epilogue (columns
    // past N only ever contribute to outputs that are not stored).
    // gemm_general_only() sends every shape to the general kernels, which otherwise only shapes beyond
    // the 32-bit offsets reach: a switch for tests and for comparing the two paths.
    const bool general_only = gemm_general_only();
    const bool fast_ok = !general_only && (K % 8 == 0) && (size_t)256 * K * 2 < ((size_t)1 << 31) &&
                         (trans_b || (size_t)K * N * 2 < ((size_t)1 << 32));
    if (fast_ok) {
#define TYR_GEMM_FAST(TB, KT)                                                                     \
        do {                                                                                      \
            static const hipError_t attr = hipFuncSetAttribute(                                   \
                reinterpret_cast<const void*>(&gemm_bf16_fast_kernel<TB, KT>),                    \
                hipFuncAttributeMaxDynamicSharedMemorySize, gemm2::LDS_BYTES);                    \
            if (attr != hipSuccess) return -1;                                                    \
            hipLaunchKernelGGL((gemm_bf16_fast_kernel<TB, KT>), grid, dim3(gemm2::THREADS), gemm2::LDS_BYTES, stream, \
                               A, Bp, Cp, M, N, K, tiles_m, tiles_n, (long)stride_a, (long)stride_b,  \
                               (long)stride_c);                                                   \
        } while (0)
        const bool k_tail = K % gemm2::BK != 0;
        if (trans_b) { if (k_tail) TYR_GEMM_FAST(true, true); else TYR_GEMM_FAST(true, false); }
        else         { if (k_tail) TYR_GEMM_FAST(false, true); else TYR_GEMM_FAST(false, false); }
#undef TYR_GEMM_FAST
        return hipGetLastError() == hipSuccess ? 0 : -1;
    }
#define TYR_GEMM_LAUNCH(TB, ED)                                                                   \
    do {                                                                                          \
        static const hipError_t attr = hipFuncSetAttribute(                                       \
            reinterpret_cast<const void*>(&gemm_bf16_kernel<TB, ED>),                             \
            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);                               \
        if (attr != hipSuccess) return -1;                                                        \
        hipLaunchKernelGGL((gemm_bf16_kernel<TB, ED>), grid, block, LDS_BYTES, stream, A, Bp, Cp, \
                           M, N, K, tiles_m, tiles_n, (long)stride_a, (long)stride_b,             \
                           (long)stride_c);                                                       \
    } while (0)
    if (trans_b) { if (edge) TYR_GEMM_LAUNCH(true, true); else TYR_GEMM_LAUNCH(true, false); }
    else         { if (edge) TYR_GEMM_LAUNCH(false, true); else TYR_GEMM_LAUNCH(false, false); }
#undef TYR_GEMM_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tyr
