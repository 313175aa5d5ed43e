// FP8 (OCP E4M3) GEMM for gfx950 with per-tensor scales:
//   C[M,N] = bf16( scale * sum_k e4m3(Aq[m,k]) * e4m3(Bq[k,n]) ),  scale = scale_a * scale_b,
// f32 accumulation on the 32x32x64 F8F6F4 MFMA (both operands format E4M3, block scales off),
// the scalar applied once in the epilogue.
//
// Arithmetic contract of the reference: Tyr/GPU/Kernels/PrecisionGemm.lean:97-115,178-189
// (e4m3 x e4m3 -> f32 -> bf16) and Tyr/GPU/Kernels/GemmCommon.lean:135-144 (one scalar
// multiplied into the f32 accumulator tile before the store).
//
// Two kernels.  The general one has the skeleton of the bf16 GEMM's general kernel: 256x256 output tile per
// 4-wave workgroup, K in slices of 128 bytes, k-contiguous padded LDS rows for both operands, two LDS
// stages with register prefetch, one barrier per slice; for B stored [K,N] its loader transposes
// 16(k) x 8(n) byte blocks in registers (two levels of v_perm_b32) on the way to LDS.  The fast one
// (further down; every shape whose offsets fit 32 bits takes it) moves slices straight into LDS and runs
// the same tile with eight waves.
#include "common.hpp"
#include "launch.hpp"

namespace tyr {

namespace gemm8 {
constexpr int BM = 256, BN = 256, BK = 128;
constexpr int ROW_BYTES = BK + 16;               // 144
constexpr int TILE_BYTES = BM * ROW_BYTES;
constexpr int LDS_BYTES = 4 * TILE_BYTES;
constexpr int THREADS = 256;
constexpr int GROUP_M = 4;
}  // namespace gemm8

// 4x4 byte transpose: o[c] = {x0.byte c, x1.byte c, x2.byte c, x3.byte c}.
__device__ __forceinline__ void transpose4x4_b8(uint32_t x0, uint32_t x1, uint32_t x2, uint32_t x3,
                                                uint32_t (&o)[4]) {
    const uint32_t t0 = __builtin_amdgcn_perm(x1, x0, 0x05010400u);  // x0.b0 x1.b0 x0.b1 x1.b1
    const uint32_t t1 = __builtin_amdgcn_perm(x1, x0, 0x07030602u);  // x0.b2 x1.b2 x0.b3 x1.b3
    const uint32_t t2 = __builtin_amdgcn_perm(x3, x2, 0x05010400u);
    const uint32_t t3 = __builtin_amdgcn_perm(x3, x2, 0x07030602u);
    o[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

template <bool TRANS_B, bool EDGE>
__global__ __launch_bounds__(gemm8::THREADS) void gemm_fp8_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, int tiles_m, int tiles_n, GemmEpilogue ep) {
    const float scale = ep.scale;
    using namespace gemm8;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int t = threadIdx.x;
    const int lane = t & 63, w = t >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int wm = w >> 1, wn = w & 1;

    const uint32_t nblk = (uint32_t)tiles_m * (uint32_t)tiles_n;
    const uint32_t pid = xcd_remap(blockIdx.x, nblk);
    const uint32_t per_group = GROUP_M * (uint32_t)tiles_n;
    const uint32_t grp = pid / per_group;
    const uint32_t first_m = grp * GROUP_M;
    const uint32_t gsz = min((uint32_t)tiles_m - first_m, (uint32_t)GROUP_M);
    const int tm = (int)(first_m + (pid % per_group) % gsz);
    const int tn = (int)((pid % per_group) / gsz);
    const int m0 = tm * BM, n0 = tn * BN;

    u32x4 ra[8];
    u32x4 rb[8];   // TRANS_B: 8 chunks of 16 B.  Otherwise viewed as 16 rows x 8 B.

    auto load_slice = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = t + THREADS * i;
            const int row = c >> 3, kc = c & 7;
            const int gm = m0 + row, gk = k0 + kc * 16;
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
                const int gn = n0 + row, gk = k0 + kc * 16;
                if (!EDGE || (gn < N && gk < K))
                    rb[i] = ld_global_16(B + (size_t)gn * K + gk);
                else
                    rb[i] = u32x4{0, 0, 0, 0};
            }
        } else {
            const int kb = t & 7, nb = t >> 3;
            const int gn = n0 + nb * 8;
#pragma unroll
            for (int i = 0; i < 8; ++i) {       // rows 2i and 2i+1 of the 16(k) x 8(n) block
                u32x2 lo = {0, 0}, hi = {0, 0};
                const int gk = k0 + kb * 16 + 2 * i;
                if (!EDGE || (gk < K && gn < N)) lo = ld_global_8(B + (size_t)gk * N + gn);
                if (!EDGE || (gk + 1 < K && gn < N)) hi = ld_global_8(B + (size_t)(gk + 1) * N + gn);
                rb[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
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
            // row k (0..15) of the block: dwords (n0..3, n4..7) = rb[k/2][2*(k&1) + {0,1}]
            u32x4 out[8];
#pragma unroll
            for (int h = 0; h < 2; ++h) {          // n half: columns 4h..4h+3
#pragma unroll
                for (int j = 0; j < 4; ++j) {      // k group: rows 4j..4j+3 -> output dword j
                    uint32_t o[4];
                    transpose4x4_b8(rb[2 * j][h], rb[2 * j][2 + h], rb[2 * j + 1][h], rb[2 * j + 1][2 + h], o);
#pragma unroll
                    for (int c = 0; c < 4; ++c) out[4 * h + c][j] = o[c];
                }
            }
#pragma unroll
            for (int nn = 0; nn < 8; ++nn)
                *reinterpret_cast<u32x4*>(Bs + (nb * 8 + nn) * ROW_BYTES + kb * 16) = out[nn];
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

    const int a_off = (wm * 128 + r) * ROW_BYTES + g * 32;
    const int b_off = (wn * 128 + r) * ROW_BYTES + g * 32;

    for (int kt = 0; kt < KT; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < KT) load_slice((kt + 1) * BK);

        const unsigned char* As = lds + stage * 2 * TILE_BYTES + a_off;
        const unsigned char* Bs = lds + stage * 2 * TILE_BYTES + TILE_BYTES + b_off;
#pragma unroll
        for (int s = 0; s < BK / 64; ++s) {
            i32x8 af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32x4 a0 = *reinterpret_cast<const u32x4*>(As + i * 32 * ROW_BYTES + s * 64);
                const u32x4 a1 = *reinterpret_cast<const u32x4*>(As + i * 32 * ROW_BYTES + s * 64 + 16);
                const u32x4 b0 = *reinterpret_cast<const u32x4*>(Bs + i * 32 * ROW_BYTES + s * 64);
                const u32x4 b1 = *reinterpret_cast<const u32x4*>(Bs + i * 32 * ROW_BYTES + s * 64 + 16);
                af[i] = i32x8{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                bf[i] = i32x8{(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mfma_32x32x64_e4m3(bf[j], af[i], acc[i][j]);
        }

        if (kt + 1 < KT) store_slice(stage ^ 1);
        __syncthreads();
    }

    if (!ep.plain_bf16()) {
        store_quadrant_ex(acc, ep, C, M, N, m0 + wm * 128, n0 + wn * 128, lane);
        return;
    }
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
                v.x = pack_bf16(acc[i][j][q4 * 4 + 0] * scale, acc[i][j][q4 * 4 + 1] * scale);
                v.y = pack_bf16(acc[i][j][q4 * 4 + 2] * scale, acc[i][j][q4 * 4 + 3] * scale);
                st_global_8(crow + gn, v);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// Fast path for K % 16 == 0 (any M; N % 16 == 0; a last slice shorter than 128 is zero-filled): slices go from global memory straight
// into LDS, unpadded rows with XOR-swizzled 16-byte chunks; a [K,N] B stays row-major in LDS and
// its fragments (32 consecutive k for one n) are gathered with the byte-transposing LDS read.
// Eight waves, two per SIMD: wave (wm, wn) owns 128 rows x 64 columns of the tile (4 x 2 MFMA tiles, 128 accumulator
// registers), so that what one wave waits for (LDS fragments, the slice barrier) is covered by the other's MFMAs.
namespace gemm8f {
constexpr int BM = 256, BN = 256, BK = 128, THREADS = 512;
constexpr int A_TILE = BM * BK;                      // 32 KiB: [256 m][8 chunks]
constexpr int B_TILE = BN * BK;                      // 32 KiB: [128 k][16 chunks] or [256 n][8 chunks]
constexpr int STAGE = A_TILE + B_TILE;
constexpr int LDS_BYTES = 2 * STAGE;
constexpr int GROUP_M = 4;
}  // namespace gemm8f

template <bool TRANS_B, bool K_TAIL>
__global__ __launch_bounds__(gemm8f::THREADS, 1) void gemm_fp8_fast_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ B, uint16_t* __restrict__ C,
    int M, int N, int K, int tiles_m, int tiles_n, GemmEpilogue ep) {
    const float scale = ep.scale;
    using namespace gemm8f;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int t = threadIdx.x;
    const int lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6);
    const int r = lane & 31, g = lane >> 5;
    const int wm = w >> 2, wn = w & 3;

    const uint32_t nblk = (uint32_t)tiles_m * (uint32_t)tiles_n;
    const uint32_t pid = xcd_remap(blockIdx.x, nblk);
    const uint32_t per_group = GROUP_M * (uint32_t)tiles_n;
    const uint32_t grp = pid / per_group;
    const uint32_t first_m = grp * GROUP_M;
    const uint32_t gsz = min((uint32_t)tiles_m - first_m, (uint32_t)GROUP_M);
    const int tm = (int)(first_m + (pid % per_group) % gsz);
    const int tn = (int)((pid % per_group) / gsz);
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> LDS requests (4 instructions of 1 KiB per wave and operand tile).
    // A (and B when TRANS_B): 8 rows of 128 B per instruction, chunk c of row m at c ^ ((m>>1)&7).
    // B when !TRANS_B: 4 rows of 256 B per instruction, chunk c of row k at c ^ ((k&7)<<1).
    // (a descriptor spans the tile's rows only and stays below 2 GiB, so that the offset 2^31 given to
    //  the chunks past K of a ragged last slice is out of range whatever is added to it; the [K,N] B
    //  descriptor is shifted down by 3072 bytes: with few columns a row is shorter than the kilobytes taken
    //  off the per-lane offsets below, and those must not go negative)
    const u32x4 a_rsrc = make_raw_rsrc(A + (size_t)m0 * K, (uint32_t)((size_t)min(M - m0, BM) * K));
    const u32x4 b_rsrc = TRANS_B
        ? make_raw_rsrc(B + (size_t)n0 * K, (uint32_t)((size_t)min(N - n0, BN) * K))
        : make_raw_rsrc(B + n0 - 3072, (uint32_t)min((size_t)K * N - n0 + 3072, (size_t)0xffffffffu));
    int a_voff[4], b_voff[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const int row = (w * 4 + m) * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        a_voff[m] = row * K + c * 16 - 1024 * m;
        if (TRANS_B) {
            b_voff[m] = row * K + c * 16 - 1024 * m;
        } else {
            const int krow = (w * 4 + m) * 4 + (lane >> 4);
            const int cb = (lane & 15) ^ ((krow & 7) << 1);
            b_voff[m] = krow * N + cb * 16 - 1024 * m + 3072;
        }
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const uint32_t wave_dst = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)w * 4096u);
    const int KT = (K + BK - 1) / BK;
    auto issue = [&](int st, int kt, int part) {         // part 0: the A tile, 1: the B tile
        const int a_soff = kt * BK;
        const int b_soff = TRANS_B ? kt * BK : kt * BK * N;
        const uint32_t dst = wave_dst + (uint32_t)st * STAGE;
        int av[4] = {a_voff[0], a_voff[1], a_voff[2], a_voff[3]};
        int bv[4] = {b_voff[0], b_voff[1], b_voff[2], b_voff[3]};
        if (K_TAIL && kt == KT - 1) {
            // ragged last slice (K % 16 == 0): the 16-byte chunks of a row at k >= K belong to the next
            // row and must read as zeros; rows k >= K of a [K,N] B are past its descriptor already
            const int chunks = (K - kt * BK) >> 4;
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

    // ---- fragment addresses.  k-step s covers bytes [64s, 64s+64) of a row; lane group g takes
    // the 32 bytes at 64s + 32g, i.e. chunks 4s + 2g and 4s + 2g + 1.
    int a_roff[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int h = 0; h < 2; ++h)
            a_roff[s][h] = (wm * 128 + r) * 128 + (((4 * s + 2 * g + h) ^ ((r >> 1) & 7)) * 16);
    int b_roff[4];    // TRANS_B: [s][h] like A.  Otherwise [jt] (two used): source-lane address for n tile jt.
    if (TRANS_B) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                b_roff[2 * s + h] = A_TILE + (wn * 64 + r) * 128 + (((4 * s + 2 * g + h) ^ ((r >> 1) & 7)) * 16);
    } else {
        // As a source lane of the byte-transposing read: k row 32(b/2) + (lane%16)/2 (+64s + 8h),
        // 8 bytes at n = wn*64 + 32jt + 16(b&1) + 8(lane%2).
        const int i16 = lane & 15, b16 = lane >> 4;
        const int js = i16 >> 1, qs = i16 & 1;
        const int krow = 32 * (b16 >> 1) + js;
#pragma unroll
        for (int jt = 0; jt < 2; ++jt) {
            const int c = wn * 4 + 2 * jt + (b16 & 1);
            b_roff[jt] = A_TILE + krow * 256 + ((c ^ (js << 1)) * 16) + qs * 8;
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

    issue(0, 0, 0);
    issue(0, 0, 1);
    wait_vmcnt0();
    __syncthreads();

    // Per slice: k-step 0 requests the next slice and reads the fragments of k-step 1; before the last MFMA row of
    // k-step 1 the workgroup waits for the requests, synchronises and reads the first fragments of the next slice.
    // The wait stands as late as the fragment reads behind it allow: the slice requests then have almost a whole slice
    // to land (after the first MFMA row of k-step 1, where it stood first, 8192^3 took 6 % longer: a fifth of the
    // requests miss the L2 and arrive later than that).  Requests and fragment reads are dealt out between the MFMA
    // rows (2 MFMAs, 128 cycles each) and the scheduling barriers keep that order.
    // (Past the last slice the requests and reads touch the idle stage / stale data and are never used.)
    i32x8 af[2][4], bf[2][2];
    auto read_a = [&](const unsigned char* St, int s, int i, i32x8& a) {
        const u32x4 x0 = *reinterpret_cast<const u32x4*>(St + a_roff[s][0] + i * 32 * 128);
        const u32x4 x1 = *reinterpret_cast<const u32x4*>(St + a_roff[s][1] + i * 32 * 128);
        a = i32x8{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
    };
    auto read_b = [&](const unsigned char* St, int s, int j, i32x8& b) {
        if (TRANS_B) {
            const u32x4 x0 = *reinterpret_cast<const u32x4*>(St + b_roff[2 * s] + j * 32 * 128);
            const u32x4 x1 = *reinterpret_cast<const u32x4*>(St + b_roff[2 * s + 1] + j * 32 * 128);
            b = i32x8{(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w, (int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
        } else {
            const unsigned char* p = St + b_roff[j] + s * 64 * 256;
            const u32x2 y0 = ds_read_tr8(p);
            const u32x2 y1 = ds_read_tr8(p + 8 * 256);
            const u32x2 y2 = ds_read_tr8(p + 16 * 256);
            const u32x2 y3 = ds_read_tr8(p + 24 * 256);
            b = i32x8{(int)y0.x, (int)y0.y, (int)y1.x, (int)y1.y, (int)y2.x, (int)y2.y, (int)y3.x, (int)y3.y};
        }
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) read_a(lds, 0, i, af[0][i]);
#pragma unroll
    for (int j = 0; j < 2; ++j) read_b(lds, 0, j, bf[0][j]);
#define TYR_FENCE __builtin_amdgcn_sched_barrier(0)
    for (int kt = 0; kt < KT; ++kt) {
        const int st = kt & 1;
        const unsigned char* St = lds + st * STAGE;
        const unsigned char* Sn = lds + (st ^ 1) * STAGE;
        auto row = [&](int s, int i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = mfma_32x32x64_e4m3(bf[s][j], af[s][i], acc[i][j]);
        };
        // The first MFMA row goes out before any fragment of the next k-step is requested: at the top of the loop
        // the compiler waits for every LDS read in flight (it cannot count across the back edge), and with fresh
        // requests in front of that wait the wave would sit out their latency once per slice.
        issue(st ^ 1, kt + 1, 0);
        TYR_FENCE; row(0, 0); TYR_FENCE;
        read_a(St, 1, 0, af[1][0]); read_b(St, 1, 0, bf[1][0]);
        issue(st ^ 1, kt + 1, 1);
        read_b(St, 1, 1, bf[1][1]); TYR_FENCE; row(0, 1); TYR_FENCE;
        read_a(St, 1, 1, af[1][1]); TYR_FENCE; row(0, 2); TYR_FENCE;
        read_a(St, 1, 2, af[1][2]);
        read_a(St, 1, 3, af[1][3]); TYR_FENCE; row(0, 3); TYR_FENCE;
        row(1, 0); TYR_FENCE;
        row(1, 1); TYR_FENCE;
        row(1, 2); TYR_FENCE;
        wait_vmcnt0();
        __syncthreads();
        read_a(Sn, 0, 0, af[0][0]); read_b(Sn, 0, 0, bf[0][0]);
        read_b(Sn, 0, 1, bf[0][1]);
        read_a(Sn, 0, 1, af[0][1]);
        read_a(Sn, 0, 2, af[0][2]);
        read_a(Sn, 0, 3, af[0][3]); TYR_FENCE; row(1, 3); TYR_FENCE;
    }
#undef TYR_FENCE

    if (!ep.plain_bf16()) {
        store_quadrant_ex<2>(acc, ep, C, M, N, m0 + wm * 128, n0 + wn * 64, lane);
        return;
    }
    store_quadrant_bf16<2>(acc, scale, lds + w * kEpilogueScratchBytes,
                           C + (size_t)(m0 + wm * 128) * N + n0 + wn * 64, N, lane,
                           M - (m0 + wm * 128), N - (n0 + wn * 64));
}

int launch_gemm_fp8(const void* aq, const void* bq, void* c, int M, int N, int K, float scale,
                    int trans_b, const float* row_scale, const float* col_scale, int out_kind, hipStream_t stream) {
    const GemmEpilogue ep{scale, row_scale, col_scale, out_kind};
    using namespace gemm8;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const bool edge = (M % BM) || (N % BN) || (K % BK);
    dim3 grid((unsigned)(tiles_m * tiles_n)), block(THREADS);
    auto A = static_cast<const uint8_t*>(aq);
    auto Bp = static_cast<const uint8_t*>(bq);
    auto Cp = static_cast<uint16_t*>(c);
    // 32-bit buffer offsets: a 256-row panel of A (and of B^T), or all of B, must stay below 4 GiB
    // The fast kernel needs whole K slices; ragged M and N are handled by the zero fill of the
    // buffer loads and by the guarded epilogue.
    // gemm_general_only() sends every shape to the general kernels, which otherwise only
    // shapes beyond the 32-bit offsets reach: a switch for tests and for comparing the two paths.
    const bool general_only = gemm_general_only();
    const bool fast_ok = !general_only && (K % 16 == 0) && (size_t)256 * K < ((size_t)1 << 31) &&
                         (trans_b || (size_t)K * N < ((size_t)1 << 32));
    if (fast_ok) {
#define TYR_GEMM8_FAST(TB, KT)                                                                      \
        do {                                                                                      \
            static const hipError_t attr = hipFuncSetAttribute(                                   \
                reinterpret_cast<const void*>(&gemm_fp8_fast_kernel<TB, KT>),                     \
                hipFuncAttributeMaxDynamicSharedMemorySize, gemm8f::LDS_BYTES);                   \
            if (attr != hipSuccess) return -1;                                                    \
            hipLaunchKernelGGL((gemm_fp8_fast_kernel<TB, KT>), grid, dim3(gemm8f::THREADS), gemm8f::LDS_BYTES, stream, \
                               A, Bp, Cp, M, N, K, tiles_m, tiles_n, ep);                         \
        } while (0)
        const bool k_tail = K % gemm8f::BK != 0;
        if (trans_b) { if (k_tail) TYR_GEMM8_FAST(true, true); else TYR_GEMM8_FAST(true, false); }
        else         { if (k_tail) TYR_GEMM8_FAST(false, true); else TYR_GEMM8_FAST(false, false); }
#undef TYR_GEMM8_FAST
        return hipGetLastError() == hipSuccess ? 0 : -1;
    }
#define TYR_GEMM8_LAUNCH(TB, ED)                                                                  \
    do {                                                                                          \
        static const hipError_t attr = hipFuncSetAttribute(                                       \
            reinterpret_cast<const void*>(&gemm_fp8_kernel<TB, ED>),                              \
            hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);                               \
        if (attr != hipSuccess) return -1;                                                        \
        hipLaunchKernelGGL((gemm_fp8_kernel<TB, ED>), grid, block, LDS_BYTES, stream, A, Bp, Cp,  \
                           M, N, K, tiles_m, tiles_n, ep);                                        \
    } while (0)
    if (trans_b) { if (edge) TYR_GEMM8_LAUNCH(true, true); else TYR_GEMM8_LAUNCH(true, false); }
    else         { if (edge) TYR_GEMM8_LAUNCH(false, true); else TYR_GEMM8_LAUNCH(false, false); }
#undef TYR_GEMM8_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tyr
