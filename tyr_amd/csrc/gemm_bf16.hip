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
    int M, int N, int K, int tiles_m, int tiles_n) {
    using namespace gemm;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

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

int launch_gemm_bf16(const void* a, const void* b, void* c, int M, int N, int K, int trans_b,
                     hipStream_t stream) {
    using namespace gemm;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const bool edge = (M % BM) || (N % BN) || (K % BK);
    dim3 grid((unsigned)(tiles_m * tiles_n)), block(THREADS);
    auto A = static_cast<const uint16_t*>(a);
    auto Bp = static_cast<const uint16_t*>(b);
    auto Cp = static_cast<uint16_t*>(c);
#define TYR_GEMM_LAUNCH(TB, ED)                                                                   \
    do {                                                                                          \
        static const hipError_t attr = hipFuncSetAttribute(                                       \
            reinterpret_cast<const void*>(&gemm_bf16_kernel<TB, ED>),                             \
            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);                               \
        if (attr != hipSuccess) return -1;                                                        \
        hipLaunchKernelGGL((gemm_bf16_kernel<TB, ED>), grid, block, LDS_BYTES, stream, A, Bp, Cp, \
                           M, N, K, tiles_m, tiles_n);                                            \
    } while (0)
    if (trans_b) { if (edge) TYR_GEMM_LAUNCH(true, true); else TYR_GEMM_LAUNCH(true, false); }
    else         { if (edge) TYR_GEMM_LAUNCH(false, true); else TYR_GEMM_LAUNCH(false, false); }
#undef TYR_GEMM_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tyr
