// Wave-level tile vocabulary for gfx950 that programs emitted from the tile DSL are written in:
// register tiles (rt), LDS tiles (st), register / LDS vectors (rv, sv), global layouts (gl) and
// the operations of the DSL's statement set (Tyr/GPU/Codegen/IR.lean:50-189) on them.
//
// It plays the part the ThunderKittens headers play for the reference's emitter
// (Tyr/GPU/Codegen/EmitNew.lean:207-330 prints `warp::load(...)`, `warp::mma_AB(...)`, ...), but it
// is built around the 64-lane wave and the 32x32x16 bf16 MFMA, not around 32-lane warps:
//
//   * One wave owns a tile program.  A 32-thread "warp" of a reference launch maps to one wave.
//   * Register tiles are grids of 32x32 blocks.  In a block of a ROW-layout tile lane
//     l = (r = l % 32, g = l / 32) holds row r and the 16 columns 8q + 4g + x (q, x = 0..3) in slot
//     4q + x.  A COL-layout tile is the transpose of that: lane holds column r and rows 8q + 4g + x.
//   * That single layout is at once the MFMA accumulator layout (with the product issued
//     transposed, so a lane owns a row) and a legal MFMA operand layout: an operand only has to
//     agree with the other operand on which k sits in which (lane half, slot), and a ROW tile used
//     as A[M,K] and a COL tile used as B[K,N] (or a ROW tile used as B^T[N,K]) agree by
//     construction.  Products therefore read registers only, and exp(S) converted to bf16 is
//     already the operand of the next product.
//   * Row reductions are in-lane plus one exchange between the lane halves; their results live in
//     ALIGN vectors (lane holds element 32b + r).  Column reductions and row-broadcast operands
//     live in ORTHO vectors (lane holds elements 32c + 8q + 4g + x).  The emitter infers which.
//
// Everything is inline device code with compile-time indexing, so tiles stay in registers.
#pragma once

#include "../common.hpp"

namespace tyr {
namespace tile {

typedef __bf16 bf16;

// OCP E4M3 (e4m3fn: bias 7, max 448, no infinity), one byte of storage; arithmetic happens in f32.
struct fp8e4m3 {
    uint8_t bits;
};

enum class layout { row, col };
enum class vlayout { align, ortho };

struct coord {
    int b, d, r, c;
};

// Row-major contiguous 4-D global tensor (batch, depth, rows, cols).
template <typename T>
struct gl {
    T* ptr;
    int nb, nd, nr, nc;
    __device__ __forceinline__ T* at(int b, int d, int r, int c) const {
        return ptr + ((((size_t)b * nd + d) * nr + r) * (size_t)nc + c);
    }
    __device__ __forceinline__ int batch() const { return nb; }
    __device__ __forceinline__ int depth() const { return nd; }
    __device__ __forceinline__ int rows() const { return nr; }
    __device__ __forceinline__ int cols() const { return nc; }
};

template <typename T, int R, int C, layout L = layout::row>
struct rt {
    static_assert(R % 32 == 0 && C % 32 == 0, "register tiles are grids of 32x32 blocks");
    typedef T dtype;
    static constexpr int rows = R, cols = C, RB = R / 32, CB = C / 32;
    static constexpr layout lay = L;
    T data[RB][CB][16];
};

// LDS tile, row-major, rows padded by 16 bytes (32 lanes reading one column chunk of 32
// consecutive rows then spread over the banks).
// PAD: bytes of padding behind every row (a multiple of 16, so that rows stay 16-byte aligned).  Which value keeps the banks
// apart depends on how the tile is read; the emitter chooses it per tile.
template <typename T, int R, int C, int PAD = 16>
struct st {
    static_assert(PAD % 16 == 0, "rows stay 16-byte aligned");
    typedef T dtype;
    static constexpr int rows = R, cols = C, pitch = C + PAD / (int)sizeof(T);
    T data[R * pitch];
    __device__ __forceinline__ T* at(int r, int c) { return data + r * pitch + c; }
    __device__ __forceinline__ const T* at(int r, int c) const { return data + r * pitch + c; }
};

template <typename T, int N, vlayout V = vlayout::align>
struct rv {
    static_assert(N % 32 == 0, "register vectors are multiples of 32 elements");
    typedef T dtype;
    static constexpr int len = N, NB = N / 32;
    static constexpr vlayout lay = V;
    T data[NB][V == vlayout::align ? 1 : 16];
};

template <typename T, int N>
struct sv {
    typedef T dtype;
    static constexpr int len = N;
    T data[N];
};

namespace detail {
__device__ __forceinline__ int lane() { return (int)(threadIdx.x & 63); }
__device__ __forceinline__ int lr() { return lane() & 31; }
__device__ __forceinline__ int lg() { return lane() >> 5; }
// LDS traffic of one wave is ordered by the hardware; this keeps the compiler from moving
// accesses across the point where other lanes' data is consumed.
__device__ __forceinline__ void wave_fence() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
template <typename T> __device__ __forceinline__ float to_f(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f(float x) { return (T)x; }
template <> __device__ __forceinline__ float to_f<fp8e4m3>(fp8e4m3 x) { return __builtin_amdgcn_cvt_f32_fp8((int)x.bits, 0); }
// round to nearest even, saturating at +-448 (the quantisation rule of the fp8 GEMM's inputs)
template <> __device__ __forceinline__ fp8e4m3 from_f<fp8e4m3>(float x) {
    const float c = x != x ? x : fminf(fmaxf(x, -448.0f), 448.0f);
    return fp8e4m3{(uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(c, 0.0f, 0, false) & 0xff)};
}
// position of slot s of block (rb, cb) for the calling lane
template <layout L> __device__ __forceinline__ int row_of(int rb, int s) {
    return L == layout::row ? 32 * rb + lr() : 32 * rb + 8 * (s >> 2) + 4 * lg() + (s & 3);
}
template <layout L> __device__ __forceinline__ int col_of(int cb, int s) {
    return L == layout::row ? 32 * cb + 8 * (s >> 2) + 4 * lg() + (s & 3) : 32 * cb + lr();
}
__device__ __forceinline__ float lane_xor(float x, int mask) { return __shfl_xor(x, mask, 64); }
}  // namespace detail

#define TYR_TILE_FOR_BLOCKS(RT)                                      \
    _Pragma("unroll") for (int rb = 0; rb < RT::RB; ++rb)            \
    _Pragma("unroll") for (int cb = 0; cb < RT::CB; ++cb)            \
    _Pragma("unroll") for (int s = 0; s < 16; ++s)

// ---------------------------------------------------------------- operation tags
struct op_copy { static __device__ __forceinline__ float f(float x) { return x; } };
struct op_zero { static __device__ __forceinline__ float f(float) { return 0.0f; } };
struct op_one { static __device__ __forceinline__ float f(float) { return 1.0f; } };
struct op_pos_infty { static __device__ __forceinline__ float f(float) { return INFINITY; } };
struct op_neg_infty { static __device__ __forceinline__ float f(float) { return -INFINITY; } };
struct op_exp { static __device__ __forceinline__ float f(float x) { return __expf(x); } };
struct op_exp2 { static __device__ __forceinline__ float f(float x) { return exp2f(x); } };
struct op_log { static __device__ __forceinline__ float f(float x) { return __logf(x); } };
struct op_log2 { static __device__ __forceinline__ float f(float x) { return log2f(x); } };
struct op_abs { static __device__ __forceinline__ float f(float x) { return fabsf(x); } };
struct op_neg { static __device__ __forceinline__ float f(float x) { return -x; } };
struct op_relu { static __device__ __forceinline__ float f(float x) { return fmaxf(x, 0.0f); } };
struct op_sqrt { static __device__ __forceinline__ float f(float x) { return sqrtf(x); } };
struct op_rsqrt { static __device__ __forceinline__ float f(float x) { return rsqrtf(x); } };
struct op_recip { static __device__ __forceinline__ float f(float x) { return 1.0f / x; } };
struct op_square { static __device__ __forceinline__ float f(float x) { return x * x; } };
struct op_tanh { static __device__ __forceinline__ float f(float x) { return tanhf(x); } };
struct op_sigmoid { static __device__ __forceinline__ float f(float x) { return 1.0f / (1.0f + __expf(-x)); } };
struct op_silu { static __device__ __forceinline__ float f(float x) { return x / (1.0f + __expf(-x)); } };
struct op_gelu {
    static __device__ __forceinline__ float f(float x) {
        return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
    }
};
struct op_sin { static __device__ __forceinline__ float f(float x) { return sinf(x); } };
struct op_cos { static __device__ __forceinline__ float f(float x) { return cosf(x); } };

struct op_add { static __device__ __forceinline__ float f(float a, float b) { return a + b; } };
struct op_sub { static __device__ __forceinline__ float f(float a, float b) { return a - b; } };
struct op_mul { static __device__ __forceinline__ float f(float a, float b) { return a * b; } };
struct op_div { static __device__ __forceinline__ float f(float a, float b) { return a / b; } };
struct op_max { static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); } };
struct op_min { static __device__ __forceinline__ float f(float a, float b) { return fminf(a, b); } };


// keep(i, j) decides which elements survive; the others take `fill`.
struct keep_causal { static __device__ __forceinline__ bool f(int i, int j, int) { return j <= i; } };       // lower triangle incl. diagonal
struct keep_causal_t { static __device__ __forceinline__ bool f(int i, int j, int) { return i <= j; } };
struct keep_tril { static __device__ __forceinline__ bool f(int i, int j, int d) { return j <= i + d; } };
struct keep_triu { static __device__ __forceinline__ bool f(int i, int j, int d) { return j >= i + d; } };
struct keep_right_fill { static __device__ __forceinline__ bool f(int, int j, int d) { return j < d; } };      // columns >= d filled
struct keep_left_fill { static __device__ __forceinline__ bool f(int, int j, int d) { return j >= d; } };      // columns < d filled
struct keep_upper_fill { static __device__ __forceinline__ bool f(int i, int, int d) { return i >= d; } };     // rows < d filled
struct keep_lower_fill { static __device__ __forceinline__ bool f(int i, int, int d) { return i < d; } };      // rows >= d filled

namespace wave {
using namespace detail;

// ---------------------------------------------------------------- global <-> LDS
template <typename T, int R, int C, int PAD>
__device__ __forceinline__ void load(st<T, R, C, PAD>& dst, const gl<T>& src, coord at) {
    constexpr int VEC = 16 / (int)sizeof(T), CPR = C / VEC;
    static_assert(C % VEC == 0 && (R * CPR) % 64 == 0, "tile is not a whole number of 16-byte pieces per lane");
#pragma unroll
    for (int k = 0; k < R * CPR / 64; ++k) {
        const int idx = lane() + 64 * k, r = idx / CPR, c = (idx % CPR) * VEC;
        const u32x4 v = *reinterpret_cast<const u32x4*>(src.at(at.b, at.d, at.r + r, at.c + c));
        *reinterpret_cast<u32x4*>(dst.at(r, c)) = v;
    }
    wave_fence();
}
// The two halves of load(st, gl, at) with the pieces a lane moves held in registers in between:
// the emitter requests the next iteration's tile of a loop before the products of the current one.
template <typename T, int R, int C>
struct gfrag {
    static constexpr int VEC = 16 / (int)sizeof(T), CPR = C / VEC, N = R * CPR / 64;
    static_assert(C % VEC == 0 && (R * CPR) % 64 == 0, "tile is not a whole number of 16-byte pieces per lane");
    u32x4 v[N];
};
template <typename T, int R, int C>
__device__ __forceinline__ void gload(gfrag<T, R, C>& dst, const gl<T>& src, coord at) {
    typedef gfrag<T, R, C> F;
#pragma unroll
    for (int k = 0; k < F::N; ++k) {
        const int idx = lane() + 64 * k, r = idx / F::CPR, c = (idx % F::CPR) * F::VEC;
        dst.v[k] = *reinterpret_cast<const u32x4*>(src.at(at.b, at.d, at.r + r, at.c + c));
    }
}
template <typename T, int R, int C, int PAD>
__device__ __forceinline__ void sstore(st<T, R, C, PAD>& dst, const gfrag<T, R, C>& src) {
    typedef gfrag<T, R, C> F;
#pragma unroll
    for (int k = 0; k < F::N; ++k) {
        const int idx = lane() + 64 * k, r = idx / F::CPR, c = (idx % F::CPR) * F::VEC;
        *reinterpret_cast<u32x4*>(dst.at(r, c)) = src.v[k];
    }
    wave_fence();
}
template <typename T, int R, int C, int PAD>
__device__ __forceinline__ void store(const gl<T>& dst, const st<T, R, C, PAD>& src, coord at) {
    constexpr int VEC = 16 / (int)sizeof(T), CPR = C / VEC;
    static_assert(C % VEC == 0 && (R * CPR) % 64 == 0, "tile is not a whole number of 16-byte pieces per lane");
    wave_fence();
#pragma unroll
    for (int k = 0; k < R * CPR / 64; ++k) {
        const int idx = lane() + 64 * k, r = idx / CPR, c = (idx % CPR) * VEC;
        const u32x4 v = *reinterpret_cast<const u32x4*>(src.at(r, c));
        *reinterpret_cast<u32x4*>(dst.at(at.b, at.d, at.r + r, at.c + c)) = v;
    }
}
// vectors: element index = idx * N (the unit of a vector coordinate is the vector)
template <typename T, int N>
__device__ __forceinline__ void load(sv<T, N>& dst, const gl<T>& src, int idx) {
#pragma unroll
    for (int k = 0; k < (N + 63) / 64; ++k)
        if (lane() + 64 * k < N) dst.data[lane() + 64 * k] = src.ptr[(size_t)idx * N + lane() + 64 * k];
    wave_fence();
}
template <typename T, int N>
__device__ __forceinline__ void store(const gl<T>& dst, const sv<T, N>& src, int idx) {
    wave_fence();
#pragma unroll
    for (int k = 0; k < (N + 63) / 64; ++k)
        if (lane() + 64 * k < N) dst.ptr[(size_t)idx * N + lane() + 64 * k] = src.data[lane() + 64 * k];
}
template <typename T, int N>
__device__ __forceinline__ void load(sv<T, N>& dst, const gl<T>& src, coord at) {
#pragma unroll
    for (int k = 0; k < (N + 63) / 64; ++k)
        if (lane() + 64 * k < N) dst.data[lane() + 64 * k] = *src.at(at.b, at.d, at.r, at.c * N + lane() + 64 * k);
    wave_fence();
}
template <typename T, int N>
__device__ __forceinline__ void store(const gl<T>& dst, const sv<T, N>& src, coord at) {
    wave_fence();
#pragma unroll
    for (int k = 0; k < (N + 63) / 64; ++k)
        if (lane() + 64 * k < N) *dst.at(at.b, at.d, at.r, at.c * N + lane() + 64 * k) = src.data[lane() + 64 * k];
}

// atomic accumulation into global memory (f32).  Every wave that executes the statement adds.
template <int R, int C, int PAD>
__device__ __forceinline__ void store_add(const gl<float>& dst, const st<float, R, C, PAD>& src, coord at) {
    wave_fence();
#pragma unroll
    for (int k = 0; k < R * C / 64; ++k) {
        const int idx = lane() + 64 * k, r = idx / C, c = idx % C;
        atomicAdd(dst.at(at.b, at.d, at.r + r, at.c + c), *src.at(r, c));
    }
}
template <int N>
__device__ __forceinline__ void store_add(const gl<float>& dst, const sv<float, N>& src, int idx) {
    wave_fence();
#pragma unroll
    for (int k = 0; k < (N + 63) / 64; ++k)
        if (lane() + 64 * k < N) atomicAdd(dst.ptr + (size_t)idx * N + lane() + 64 * k, src.data[lane() + 64 * k]);
}
template <int N>
__device__ __forceinline__ void store_add(const gl<float>& dst, const sv<float, N>& src, coord at) {
    wave_fence();
#pragma unroll
    for (int k = 0; k < (N + 63) / 64; ++k)
        if (lane() + 64 * k < N) atomicAdd(dst.at(at.b, at.d, at.r, at.c * N + lane() + 64 * k), src.data[lane() + 64 * k]);
}

// ---------------------------------------------------------------- LDS <-> registers
namespace detail {
// The four slots 4q .. 4q+3 of a ROW tile are four consecutive columns of one row: one 4-element access.
template <typename T> struct quad { T v[4]; } __attribute__((aligned(sizeof(T) * 4 <= 16 ? sizeof(T) * 4 : 16)));
template <typename T, int RS, int R, int C, int PAD>
__device__ __forceinline__ void load_rows(rt<T, RS, C, layout::row>& dst, const st<T, R, C, PAD>& src, int row0) {
#pragma unroll
    for (int rb = 0; rb < RS / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const quad<T> v = *reinterpret_cast<const quad<T>*>(src.at(row0 + 32 * rb + lr(), 32 * cb + 8 * q + 4 * lg()));
#pragma unroll
                for (int x = 0; x < 4; ++x) dst.data[rb][cb][4 * q + x] = v.v[x];
            }
}
template <typename T, int RS, int R, int C, int PAD>
__device__ __forceinline__ void store_rows(st<T, R, C, PAD>& dst, const rt<T, RS, C, layout::row>& src, int row0) {
#pragma unroll
    for (int rb = 0; rb < RS / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                quad<T> v;
#pragma unroll
                for (int x = 0; x < 4; ++x) v.v[x] = src.data[rb][cb][4 * q + x];
                *reinterpret_cast<quad<T>*>(dst.at(row0 + 32 * rb + lr(), 32 * cb + 8 * q + 4 * lg())) = v;
            }
}
}  // namespace detail
template <typename T, int R, int C, layout L, int PAD>
__device__ __forceinline__ void load(rt<T, R, C, L>& dst, const st<T, R, C, PAD>& src) {
    typedef rt<T, R, C, L> RT;
    if constexpr (L == layout::row) {
        detail::load_rows(dst, src, 0);
        return;
    }
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = *src.at(row_of<L>(rb, s), col_of<L>(cb, s));
}
// COL tiles of 2-byte elements: a lane wants 4 consecutive rows of one column per slot group, which is
// what the transposing LDS read delivers (16 lanes x 8 bytes along 4 rows in, 4 rows of one column out).
template <int R, int C, int PAD>
__device__ __forceinline__ void load(rt<bf16, R, C, layout::col>& dst, const st<bf16, R, C, PAD>& src) {
    const int i16 = lane() & 15, b16 = lane() >> 4;
    const int srow = 4 * (b16 >> 1) + (i16 >> 2), scol = 16 * (b16 & 1) + 4 * (i16 & 3);   // this lane as a source
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const bf16x4 v = ds_read_tr16(src.at(32 * rb + 8 * q + srow, 32 * cb + scol));
#pragma unroll
                for (int x = 0; x < 4; ++x) dst.data[rb][cb][4 * q + x] = v[x];
            }
}
template <typename T, int R, int C, layout L, int PAD>
__device__ __forceinline__ void store(st<T, R, C, PAD>& dst, const rt<T, R, C, L>& src) {
    typedef rt<T, R, C, L> RT;
    if constexpr (L == layout::row) {
        detail::store_rows(dst, src, 0);
        wave_fence();
        return;
    }
    TYR_TILE_FOR_BLOCKS(RT) *dst.at(row_of<L>(rb, s), col_of<L>(cb, s)) = src.data[rb][cb][s];
    wave_fence();
}
template <typename T, int N, vlayout V>
__device__ __forceinline__ void load(rv<T, N, V>& dst, const sv<T, N>& src) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b) {
        if (V == vlayout::align) {
            dst.data[b][0] = src.data[32 * b + lr()];
        } else {
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[b][s] = src.data[col_of<layout::row>(b, s)];
        }
    }
}
template <typename T, int N, vlayout V>
__device__ __forceinline__ void store(sv<T, N>& dst, const rv<T, N, V>& src) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b) {
        if (V == vlayout::align) {
            if (lg() == 0) dst.data[32 * b + lr()] = src.data[b][0];
        } else {
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (lr() == 0) dst.data[col_of<layout::row>(b, s)] = src.data[b][s];
        }
    }
    wave_fence();
}

// ---------------------------------------------------------------- products
// D = A B + C on the 32x32x16 bf16 MFMA.  The product is issued transposed (the B fragment as
// the MFMA's row operand) so that the accumulator comes out in ROW layout.
namespace detail {
template <typename TA, typename TB>
__device__ __forceinline__ void mfma_block(float (&d)[16], const TA (&a)[16], const TB (&b)[16]) {
    static_assert(sizeof(TA) == 2 && sizeof(TB) == 2, "products take bf16 operands");
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = d[e];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        bf16x8 fa, fb;
#pragma unroll
        for (int e = 0; e < 8; ++e) { fa[e] = a[8 * h + e]; fb[e] = b[8 * h + e]; }
        acc = mfma_32x32x16_bf16(fb, fa, acc);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) d[e] = acc[e];
}
}  // namespace detail

#define TYR_TILE_MMA(NAME, ATYPE, BTYPE, KDIM, AIDX, BIDX)                                          \
    template <int M, int N, int K>                                                                  \
    __device__ __forceinline__ void NAME(rt<float, M, N, layout::row>& d, const ATYPE& a,           \
                                         const BTYPE& b, const rt<float, M, N, layout::row>& c) {   \
        _Pragma("unroll") for (int mb = 0; mb < M / 32; ++mb)                                       \
        _Pragma("unroll") for (int nb = 0; nb < N / 32; ++nb) {                                     \
            float acc[16];                                                                          \
            _Pragma("unroll") for (int e = 0; e < 16; ++e) acc[e] = c.data[mb][nb][e];              \
            _Pragma("unroll") for (int kb = 0; kb < KDIM / 32; ++kb)                                \
                detail::mfma_block(acc, a.data AIDX, b.data BIDX);                                  \
            _Pragma("unroll") for (int e = 0; e < 16; ++e) d.data[mb][nb][e] = acc[e];              \
        }                                                                                           \
    }
#define TYR_TILE_COMMA ,
// A[M,K] row, B[K,N] col
TYR_TILE_MMA(mma_AB, rt<bf16 TYR_TILE_COMMA M TYR_TILE_COMMA K TYR_TILE_COMMA layout::row>,
             rt<bf16 TYR_TILE_COMMA K TYR_TILE_COMMA N TYR_TILE_COMMA layout::col>, K, [mb][kb], [kb][nb])
// A[M,K] row, B[N,K] row
TYR_TILE_MMA(mma_ABt, rt<bf16 TYR_TILE_COMMA M TYR_TILE_COMMA K TYR_TILE_COMMA layout::row>,
             rt<bf16 TYR_TILE_COMMA N TYR_TILE_COMMA K TYR_TILE_COMMA layout::row>, K, [mb][kb], [nb][kb])
// A[K,M] col, B[K,N] col
TYR_TILE_MMA(mma_AtB, rt<bf16 TYR_TILE_COMMA K TYR_TILE_COMMA M TYR_TILE_COMMA layout::col>,
             rt<bf16 TYR_TILE_COMMA K TYR_TILE_COMMA N TYR_TILE_COMMA layout::col>, K, [kb][mb], [kb][nb])
// A[K,M] col, B[N,K] row
TYR_TILE_MMA(mma_AtBt, rt<bf16 TYR_TILE_COMMA K TYR_TILE_COMMA M TYR_TILE_COMMA layout::col>,
             rt<bf16 TYR_TILE_COMMA N TYR_TILE_COMMA K TYR_TILE_COMMA layout::row>, K, [kb][mb], [nb][kb])
#undef TYR_TILE_MMA
// E4M3 operands: A[M,K] row, B[N,K] row, on the 32x32x64 MFMA (a lane's 16 bytes of two adjacent
// 32-column blocks are its 32 bytes of k; both operands use the same map).
template <int M, int N, int K>
__device__ __forceinline__ void mma_ABt(rt<float, M, N, layout::row>& d, const rt<fp8e4m3, M, K, layout::row>& a,
                                        const rt<fp8e4m3, N, K, layout::row>& b, const rt<float, M, N, layout::row>& c) {
    static_assert(K % 64 == 0, "E4M3 products consume k in steps of 64");
#pragma unroll
    for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
        for (int nb = 0; nb < N / 32; ++nb) {
            f32x16 acc;
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[e] = c.data[mb][nb][e];
#pragma unroll
            for (int kb = 0; kb < K / 32; kb += 2) {
                i32x8 fa, fb;
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int wd = 0; wd < 4; ++wd) {
                        uint32_t ua = 0, ub = 0;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            ua |= (uint32_t)a.data[mb][kb + h][4 * wd + e].bits << (8 * e);
                            ub |= (uint32_t)b.data[nb][kb + h][4 * wd + e].bits << (8 * e);
                        }
                        fa[4 * h + wd] = (int)ua;
                        fb[4 * h + wd] = (int)ub;
                    }
                acc = mfma_32x32x64_e4m3(fb, fa, acc);
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) d.data[mb][nb][e] = acc[e];
        }
}

// ---------------------------------------------------------------- element-wise
// Arithmetic is done in f32 whatever the storage type; results are rounded to the storage type.
template <typename OP, typename T, int R, int C, layout L>
__device__ __forceinline__ void unary(rt<T, R, C, L>& dst, const rt<T, R, C, L>& src) {
    typedef rt<T, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(OP::f(to_f(src.data[rb][cb][s])));
}
template <typename OP, typename T, int N, vlayout V>
__device__ __forceinline__ void unary(rv<T, N, V>& dst, const rv<T, N, V>& src) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<T>(OP::f(to_f(src.data[b][s])));
}
template <typename OP, typename T, int R, int C, layout L>
__device__ __forceinline__ void binary(rt<T, R, C, L>& dst, const rt<T, R, C, L>& a, const rt<T, R, C, L>& b) {
    typedef rt<T, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(OP::f(to_f(a.data[rb][cb][s]), to_f(b.data[rb][cb][s])));
}
template <typename OP, typename T, int N, vlayout V>
__device__ __forceinline__ void binary(rv<T, N, V>& dst, const rv<T, N, V>& a, const rv<T, N, V>& b) {
#pragma unroll
    for (int bl = 0; bl < N / 32; ++bl)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s)
            dst.data[bl][s] = from_f<T>(OP::f(to_f(a.data[bl][s]), to_f(b.data[bl][s])));
}
template <typename OP, typename T, int R, int C, layout L>
__device__ __forceinline__ void scalar(rt<T, R, C, L>& dst, const rt<T, R, C, L>& src, float k) {
    typedef rt<T, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(OP::f(to_f(src.data[rb][cb][s]), k));
}
template <typename OP, typename T, int N, vlayout V>
__device__ __forceinline__ void scalar(rv<T, N, V>& dst, const rv<T, N, V>& src, float k) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<T>(OP::f(to_f(src.data[b][s]), k));
}
// dst = a * b + c
template <typename T, int R, int C, layout L>
__device__ __forceinline__ void fma(rt<T, R, C, L>& dst, const rt<T, R, C, L>& a, const rt<T, R, C, L>& b,
                                    const rt<T, R, C, L>& c) {
    typedef rt<T, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT)
        dst.data[rb][cb][s] = from_f<T>(fmaf(to_f(a.data[rb][cb][s]), to_f(b.data[rb][cb][s]), to_f(c.data[rb][cb][s])));
}
template <typename TD, typename TS, int R, int C, layout L>
__device__ __forceinline__ void convert(rt<TD, R, C, L>& dst, const rt<TS, R, C, L>& src) {
    typedef rt<TD, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<TD>(to_f(src.data[rb][cb][s]));
}
template <typename TD, typename TS, int N, vlayout V>
__device__ __forceinline__ void convert(rv<TD, N, V>& dst, const rv<TS, N, V>& src) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<TD>(to_f(src.data[b][s]));
}
// The transpose of a ROW tile is the COL tile with the same registers (and back).
template <typename T, int R, int C>
__device__ __forceinline__ void transpose(rt<T, C, R, layout::col>& dst, const rt<T, R, C, layout::row>& src) {
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[cb][rb][s] = src.data[rb][cb][s];
}
template <typename T, int R, int C>
__device__ __forceinline__ void transpose(rt<T, C, R, layout::row>& dst, const rt<T, R, C, layout::col>& src) {
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[cb][rb][s] = src.data[rb][cb][s];
}
// Transpose that keeps the layout kind: through an LDS tile of the source's shape.
template <typename T, int R, int C, layout L, int PAD>
__device__ __forceinline__ void transpose(rt<T, C, R, L>& dst, const rt<T, R, C, L>& src, st<T, R, C, PAD>& scratch) {
    store(scratch, src);
    typedef rt<T, C, R, L> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = *scratch.at(col_of<L>(cb, s), row_of<L>(rb, s));
    wave_fence();
}
// Same matrix, other layout: through an LDS tile the caller provides.
template <typename T, int R, int C, layout LD, layout LS, int PAD>
__device__ __forceinline__ void swap_layout(rt<T, R, C, LD>& dst, const rt<T, R, C, LS>& src, st<T, R, C, PAD>& scratch) {
    store(scratch, src);
    load(dst, scratch);
    wave_fence();
}

// column ranges at multiples of 32
template <int START, typename T, int R, int C, int CS, layout L>
__device__ __forceinline__ void slice_cols(rt<T, R, CS, L>& dst, const rt<T, R, C, L>& src) {
    static_assert(START % 32 == 0 && START + CS <= C, "column slices start at multiples of 32");
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < CS / 32; ++cb)
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[rb][cb][s] = src.data[rb][START / 32 + cb][s];
}
template <int START, typename T, int R, int C, int RS, layout L>
__device__ __forceinline__ void slice_rows(rt<T, RS, C, L>& dst, const rt<T, R, C, L>& src) {
    static_assert(START % 32 == 0 && START + RS <= R, "row slices start at multiples of 32");
#pragma unroll
    for (int rb = 0; rb < RS / 32; ++rb)
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[rb][cb][s] = src.data[START / 32 + rb][cb][s];
}
template <typename T, int R, int CL, int CR, layout L>
__device__ __forceinline__ void concat_cols(rt<T, R, CL + CR, L>& dst, const rt<T, R, CL, L>& left,
                                            const rt<T, R, CR, L>& right) {
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb) {
#pragma unroll
        for (int cb = 0; cb < CL / 32; ++cb)
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[rb][cb][s] = left.data[rb][cb][s];
#pragma unroll
        for (int cb = 0; cb < CR / 32; ++cb)
#pragma unroll
            for (int s = 0; s < 16; ++s) dst.data[rb][CL / 32 + cb][s] = right.data[rb][cb][s];
    }
}

// ---------------------------------------------------------------- masks
template <typename KEEP, typename T, int R, int C, layout L>
__device__ __forceinline__ void mask(rt<T, R, C, L>& dst, const rt<T, R, C, L>& src, float fill, int d = 0) {
    typedef rt<T, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT)
        dst.data[rb][cb][s] = KEEP::f(row_of<L>(rb, s), col_of<L>(cb, s), d) ? src.data[rb][cb][s] : from_f<T>(fill);
}
// rows < r0 of columns >= c0 take `fill`
template <typename T, int R, int C, layout L>
__device__ __forceinline__ void mask_upper_right(rt<T, R, C, L>& dst, const rt<T, R, C, L>& src, float fill, int r0, int c0) {
    typedef rt<T, R, C, L> RT;
    TYR_TILE_FOR_BLOCKS(RT)
        dst.data[rb][cb][s] = (row_of<L>(rb, s) < r0 && col_of<L>(cb, s) >= c0) ? from_f<T>(fill) : src.data[rb][cb][s];
}
// v[i] = start + step * i ;  v[i] = x
template <typename T, int N, vlayout V>
__device__ __forceinline__ void iota(rv<T, N, V>& dst, float start, float step) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s) {
            const int i = V == vlayout::align ? 32 * b + lr() : col_of<layout::row>(b, s);
            dst.data[b][s] = from_f<T>(start + step * (float)i);
        }
}
template <typename T, int N, vlayout V>
__device__ __forceinline__ void fill(rv<T, N, V>& dst, float x) {
#pragma unroll
    for (int b = 0; b < N / 32; ++b)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<T>(x);
}

// ---------------------------------------------------------------- reductions and broadcasts (ROW tiles)
// row_reduce: dst[i] = OP over j of src[i][j]  (ALIGN vector);  with `accum`: OP(that, accum[i]).
template <typename OP, typename T, int R, int C>
__device__ __forceinline__ void row_reduce(rv<T, R, vlayout::align>& dst, const rt<T, R, C, layout::row>& src) {
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb) {
        float acc = to_f(src.data[rb][0][0]);
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int s = (cb == 0 ? 1 : 0); s < 16; ++s) acc = OP::f(acc, to_f(src.data[rb][cb][s]));
        dst.data[rb][0] = from_f<T>(OP::f(acc, xor32(acc)));
    }
}
template <typename OP, typename T, int R, int C>
__device__ __forceinline__ void row_reduce(rv<T, R, vlayout::align>& dst, const rt<T, R, C, layout::row>& src,
                                           const rv<T, R, vlayout::align>& accum) {
    rv<T, R, vlayout::align> tmp;
    row_reduce<OP>(tmp, src);
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb) dst.data[rb][0] = from_f<T>(OP::f(to_f(tmp.data[rb][0]), to_f(accum.data[rb][0])));
}
// col_reduce: dst[j] = OP over i of src[i][j]  (ORTHO vector)
template <typename OP, typename T, int R, int C>
__device__ __forceinline__ void col_reduce(rv<T, C, vlayout::ortho>& dst, const rt<T, R, C, layout::row>& src) {
#pragma unroll
    for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            float acc = to_f(src.data[0][cb][s]);
#pragma unroll
            for (int rb = 1; rb < R / 32; ++rb) acc = OP::f(acc, to_f(src.data[rb][cb][s]));
#pragma unroll
            for (int m = 1; m < 32; m <<= 1) acc = OP::f(acc, lane_xor(acc, m));
            dst.data[cb][s] = from_f<T>(acc);
        }
}
template <typename OP, typename T, int R, int C>
__device__ __forceinline__ void col_reduce(rv<T, C, vlayout::ortho>& dst, const rt<T, R, C, layout::row>& src,
                                           const rv<T, C, vlayout::ortho>& accum) {
    rv<T, C, vlayout::ortho> tmp;
    col_reduce<OP>(tmp, src);
#pragma unroll
    for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
        for (int s = 0; s < 16; ++s) dst.data[cb][s] = from_f<T>(OP::f(to_f(tmp.data[cb][s]), to_f(accum.data[cb][s])));
}
// dst[i][j] = OP(src[i][j], v[i])   (the DSL's *Col operations: v is a column vector)
template <typename OP, typename T, typename TV, int R, int C>
__device__ __forceinline__ void col_broadcast(rt<T, R, C, layout::row>& dst, const rt<T, R, C, layout::row>& src,
                                              const rv<TV, R, vlayout::align>& v) {
    typedef rt<T, R, C, layout::row> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(OP::f(to_f(src.data[rb][cb][s]), to_f(v.data[rb][0])));
}
// dst[i][j] = OP(src[i][j], v[j])   (the DSL's *Row operations: v is a row vector)
template <typename OP, typename T, typename TV, int R, int C>
__device__ __forceinline__ void row_broadcast(rt<T, R, C, layout::row>& dst, const rt<T, R, C, layout::row>& src,
                                              const rv<TV, C, vlayout::ortho>& v) {
    typedef rt<T, R, C, layout::row> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(OP::f(to_f(src.data[rb][cb][s]), to_f(v.data[cb][s])));
}
// dst[i][j] = v[i] / v[j]
template <typename T, typename TV, int R, int C>
__device__ __forceinline__ void broadcast_col(rt<T, R, C, layout::row>& dst, const rv<TV, R, vlayout::align>& v) {
    typedef rt<T, R, C, layout::row> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(to_f(v.data[rb][0]));
}
template <typename T, typename TV, int R, int C>
__device__ __forceinline__ void broadcast_row(rt<T, R, C, layout::row>& dst, const rv<TV, C, vlayout::ortho>& v) {
    typedef rt<T, R, C, layout::row> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(to_f(v.data[cb][s]));
}
// dst[i][j] = a[i] * b[j]
template <typename T, typename TV, int R, int C>
__device__ __forceinline__ void outer(rt<T, R, C, layout::row>& dst, const rv<TV, R, vlayout::align>& a,
                                      const rv<TV, C, vlayout::ortho>& b) {
    typedef rt<T, R, C, layout::row> RT;
    TYR_TILE_FOR_BLOCKS(RT) dst.data[rb][cb][s] = from_f<T>(to_f(a.data[rb][0]) * to_f(b.data[cb][s]));
}

// ---------------------------------------------------------------- the online-softmax step as one operation
// What the statement sequence of the reference's `onlineSoftmax` macro (Tyr/GPU/Codegen/Macros.lean:121-147), optionally
// preceded by a multiplication of the scores by a positive constant, computes:
//     prev = mx;  mx = max(mx, rowmax(c s));  scl = exp(prev - mx);  o *= scl;  sum *= scl;
//     s = exp(c s - mx);  sum = rowsum(s) + sum
// with the same values left in every operand.  Fused, the scale and the change to base 2 fold into one multiply-add per
// score in front of the exponential instruction, and the accumulator is only rescaled when some row's maximum moved
// (scl is exactly 1 otherwise).  The emitter substitutes this call where it recognises the sequence.
template <int R, int C, int CO>
__device__ __forceinline__ void online_softmax(rt<float, R, C, layout::row>& s, rt<float, R, CO, layout::row>& o,
                                               rv<float, R, vlayout::align>& mx, rv<float, R, vlayout::align>& sum,
                                               rv<float, R, vlayout::align>& prev, rv<float, R, vlayout::align>& scl, float c) {
    constexpr float kLog2e = 1.4426950408889634f;
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb) {
        float m = s.data[rb][0][0];
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int e = (cb == 0 ? 1 : 0); e < 16; ++e) m = fmaxf(m, s.data[rb][cb][e]);
        m = fmaxf(m, xor32(m)) * c;                  // c > 0: the maximum of the scaled scores
        const float old = mx.data[rb][0];
        const float now = fmaxf(old, m);
        const float f = __expf(old - now);
        prev.data[rb][0] = old;
        mx.data[rb][0] = now;
        scl.data[rb][0] = f;
        if (__builtin_amdgcn_ballot_w64(f != 1.0f) != 0) {
#pragma unroll
            for (int cb = 0; cb < CO / 32; ++cb)
#pragma unroll
                for (int e = 0; e < 16; ++e) o.data[rb][cb][e] *= f;
        }
        const float c2 = c * kLog2e, m2 = now * kLog2e;
        float acc = 0.0f;
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s.data[rb][cb][e], c2, -m2));
                s.data[rb][cb][e] = p;
                acc += p;
            }
        sum.data[rb][0] = (acc + xor32(acc)) + sum.data[rb][0] * f;
    }
}

// ---------------------------------------------------------------- full reductions and scans (vectors, tiles)
// The reference's IR has a third axis, "Full" (Tyr/GPU/Codegen/AST.lean:54-63; printed as the unprefixed warp::max /
// warp::sum / warp::cumsum, i.e. the vector forms): the reduction of every element, here left in every element of the
// destination vector, and the running reduction along a vector.
namespace detail {
// OP over the `len` elements of a vector, on every lane.  ALIGN: lane (r, g) holds element 32b + r (both halves the same
// value); ORTHO: slot s of lane half g holds element 32b + 8(s/4) + 4g + s%4 (every row lane the same value).
template <typename OP, typename T, int N, vlayout V>
__device__ __forceinline__ float reduce_all(const rv<T, N, V>& src) {
    float acc = to_f(src.data[0][0]);
#pragma unroll
    for (int b = 0; b < N / 32; ++b)
#pragma unroll
        for (int s = 0; s < (V == vlayout::align ? 1 : 16); ++s)
            if (b != 0 || s != 0) acc = OP::f(acc, to_f(src.data[b][s]));
    if constexpr (V == vlayout::align) {
#pragma unroll
        for (int m = 1; m < 32; m <<= 1) acc = OP::f(acc, lane_xor(acc, m));
    } else {
        acc = OP::f(acc, xor32(acc));
    }
    return acc;
}
}  // namespace detail
template <typename OP, typename T, int ND, vlayout VD, int N, vlayout V>
__device__ __forceinline__ void full_reduce(rv<T, ND, VD>& dst, const rv<T, N, V>& src) {
    const float x = detail::reduce_all<OP>(src);
#pragma unroll
    for (int b = 0; b < ND / 32; ++b)
#pragma unroll
        for (int s = 0; s < (VD == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<T>(x);
}
template <typename OP, typename T, int ND, vlayout VD, int N, vlayout V>
__device__ __forceinline__ void full_reduce(rv<T, ND, VD>& dst, const rv<T, N, V>& src, const rv<T, ND, VD>& accum) {
    const float x = detail::reduce_all<OP>(src);
#pragma unroll
    for (int b = 0; b < ND / 32; ++b)
#pragma unroll
        for (int s = 0; s < (VD == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<T>(OP::f(x, to_f(accum.data[b][s])));
}
// every element of a ROW tile: rows first, then the row results
template <typename OP, typename T, int ND, vlayout VD, int R, int C>
__device__ __forceinline__ void full_reduce(rv<T, ND, VD>& dst, const rt<T, R, C, layout::row>& src) {
    rv<float, R, vlayout::align> rows;
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb) {
        float acc = to_f(src.data[rb][0][0]);
#pragma unroll
        for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
            for (int s = (cb == 0 ? 1 : 0); s < 16; ++s) acc = OP::f(acc, to_f(src.data[rb][cb][s]));
        rows.data[rb][0] = OP::f(acc, xor32(acc));
    }
    const float x = detail::reduce_all<OP>(rows);
#pragma unroll
    for (int b = 0; b < ND / 32; ++b)
#pragma unroll
        for (int s = 0; s < (VD == vlayout::align ? 1 : 16); ++s) dst.data[b][s] = from_f<T>(x);
}
// dst[i] = OP over i' <= i of src[i'] along an ALIGN vector: a scan over the 32 row lanes, carried from block to block
template <typename OP, typename T, int N>
__device__ __forceinline__ void full_scan(rv<T, N, vlayout::align>& dst, const rv<T, N, vlayout::align>& src) {
    float carry = 0.0f;
#pragma unroll
    for (int b = 0; b < N / 32; ++b) {
        float x = to_f(src.data[b][0]);
#pragma unroll
        for (int d = 1; d < 32; d <<= 1) {
            const float up = __shfl_up(x, d, 32);
            if (lr() >= d) x = OP::f(up, x);
        }
        if (b > 0) x = OP::f(carry, x);
        dst.data[b][0] = from_f<T>(x);
        carry = __shfl(x, 31, 32);
    }
}

// ---------------------------------------------------------------- scans (ROW tiles)
// row_scan: dst[i][j] = OP over j' <= j of src[i][j'].  A lane owns the 4-column groups 8q + 4g of
// its row; group totals are exchanged with the other lane half and prefixed in column order.
template <typename OP, typename T, int R, int C>
__device__ __forceinline__ void row_scan(rt<T, R, C, layout::row>& dst, const rt<T, R, C, layout::row>& src) {
    constexpr int NG = C / 8;                        // groups per lane per row
#pragma unroll
    for (int rb = 0; rb < R / 32; ++rb) {
        float v[NG][4], own[NG], other[NG];
#pragma unroll
        for (int k = 0; k < NG; ++k) {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const float e = to_f(src.data[rb][k >> 2][4 * (k & 3) + x]);
                v[k][x] = x == 0 ? e : OP::f(v[k][x - 1], e);
            }
            own[k] = v[k][3];
            other[k] = xor32(own[k]);
        }
        float base = 0.0f;
        bool have = false;                           // `base` holds a value (no identity element is assumed)
#pragma unroll
        for (int k = 0; k < NG; ++k) {
            const float lo = lg() == 0 ? own[k] : other[k], hi = lg() == 0 ? other[k] : own[k];
            // prefix in front of this lane's group: everything before (k), plus the low half's group for the high half
            float pre = base;
            bool pre_have = have;
            if (lg() == 1) { pre = have ? OP::f(base, lo) : lo; pre_have = true; }
#pragma unroll
            for (int x = 0; x < 4; ++x)
                dst.data[rb][k >> 2][4 * (k & 3) + x] = from_f<T>(pre_have ? OP::f(pre, v[k][x]) : v[k][x]);
            base = have ? OP::f(OP::f(base, lo), hi) : OP::f(lo, hi);
            have = true;
        }
    }
}
// col_scan: dst[i][j] = OP over i' <= i of src[i'][j]: a scan over the 32 lanes of a half, carried
// from one row block to the next.
template <typename OP, typename T, int R, int C>
__device__ __forceinline__ void col_scan(rt<T, R, C, layout::row>& dst, const rt<T, R, C, layout::row>& src) {
#pragma unroll
    for (int cb = 0; cb < C / 32; ++cb)
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            float carry = 0.0f;
#pragma unroll
            for (int rb = 0; rb < R / 32; ++rb) {
                float x = to_f(src.data[rb][cb][s]);
#pragma unroll
                for (int d = 1; d < 32; d <<= 1) {
                    const float up = __shfl_up(x, d, 32);
                    if (lr() >= d) x = OP::f(up, x);
                }
                if (rb > 0) x = OP::f(carry, x);
                dst.data[rb][cb][s] = from_f<T>(x);
                carry = __shfl(x, 31, 32);           // the block's last row, within this lane half
            }
        }
}

__device__ __forceinline__ void sync() { __syncthreads(); }

// ---------------------------------------------------------------- wave groups
// A program whose register tiles do not fit one wave is run by a group of W waves: tiles and ALIGN
// vectors that are tied to one another through their rows are cut into W row slices, wave w owning
// rows [w R/W, (w+1) R/W); everything else (B operands, ORTHO vectors) is common to the group.  The
// pieces below are what the emitter prints for such a program.
__device__ __forceinline__ int index() { return (int)(threadIdx.x >> 6); }

// global <-> LDS, the group sharing the tile: wave `part` of `nparts` moves its share of the rows
template <typename T, int R, int C, int PAD>
__device__ __forceinline__ void load_part(st<T, R, C, PAD>& dst, const gl<T>& src, coord at, int part, int nparts) {
    constexpr int VEC = 16 / (int)sizeof(T), CPR = C / VEC;
    static_assert(C % VEC == 0, "rows are whole 16-byte pieces");
    for (int idx = part * 64 + lane(); idx < R * CPR; idx += 64 * nparts) {
        const int r = idx / CPR, c = (idx % CPR) * VEC;
        *reinterpret_cast<u32x4*>(dst.at(r, c)) = *reinterpret_cast<const u32x4*>(src.at(at.b, at.d, at.r + r, at.c + c));
    }
    wave_fence();
}
template <typename T, int R, int C, int PAD>
__device__ __forceinline__ void store_part(const gl<T>& dst, const st<T, R, C, PAD>& src, coord at, int part, int nparts) {
    constexpr int VEC = 16 / (int)sizeof(T), CPR = C / VEC;
    static_assert(C % VEC == 0, "rows are whole 16-byte pieces");
    wave_fence();
    for (int idx = part * 64 + lane(); idx < R * CPR; idx += 64 * nparts) {
        const int r = idx / CPR, c = (idx % CPR) * VEC;
        *reinterpret_cast<u32x4*>(dst.at(at.b, at.d, at.r + r, at.c + c)) = *reinterpret_cast<const u32x4*>(src.at(r, c));
    }
}
// The two halves of load_part with the pieces a lane moves held in registers in between (wave `part` of W
// takes pieces part*64 + lane, + 64 W, ...): the next iteration's tile is requested before the products of
// the current one.
template <typename T, int R, int C, int W>
struct gfrag_part {
    static constexpr int VEC = 16 / (int)sizeof(T), CPR = C / VEC, N = R * CPR / (64 * W);
    static_assert(C % VEC == 0 && (R * CPR) % (64 * W) == 0, "the waves share the tile's 16-byte pieces evenly");
    u32x4 v[N];
};
template <typename T, int R, int C, int W>
__device__ __forceinline__ void gload_part(gfrag_part<T, R, C, W>& dst, const gl<T>& src, coord at, int part) {
    typedef gfrag_part<T, R, C, W> F;
#pragma unroll
    for (int k = 0; k < F::N; ++k) {
        const int idx = part * 64 + lane() + 64 * W * k, r = idx / F::CPR, c = (idx % F::CPR) * F::VEC;
        dst.v[k] = *reinterpret_cast<const u32x4*>(src.at(at.b, at.d, at.r + r, at.c + c));
    }
}
template <typename T, int R, int C, int W, int PAD>
__device__ __forceinline__ void sstore_part(st<T, R, C, PAD>& dst, const gfrag_part<T, R, C, W>& src, int part) {
    typedef gfrag_part<T, R, C, W> F;
#pragma unroll
    for (int k = 0; k < F::N; ++k) {
        const int idx = part * 64 + lane() + 64 * W * k, r = idx / F::CPR, c = (idx % F::CPR) * F::VEC;
        *reinterpret_cast<u32x4*>(dst.at(r, c)) = src.v[k];
    }
    wave_fence();
}
// a wave's row slice of an LDS tile / vector <-> registers
template <typename T, int RS, int R, int C, int PAD>
__device__ __forceinline__ void load(rt<T, RS, C, layout::row>& dst, const st<T, R, C, PAD>& src, int row0) {
    static_assert(RS <= R, "a slice is no taller than its tile");
    detail::load_rows(dst, src, row0);
}
template <typename T, int RS, int R, int C, int PAD>
__device__ __forceinline__ void store(st<T, R, C, PAD>& dst, const rt<T, RS, C, layout::row>& src, int row0) {
    static_assert(RS <= R, "a slice is no taller than its tile");
    detail::store_rows(dst, src, row0);
    wave_fence();
}
template <typename T, int NS, int N>
__device__ __forceinline__ void load(rv<T, NS, vlayout::align>& dst, const sv<T, N>& src, int off) {
#pragma unroll
    for (int b = 0; b < NS / 32; ++b) dst.data[b][0] = src.data[off + 32 * b + lr()];
}
template <typename T, int NS, int N>
__device__ __forceinline__ void store(sv<T, N>& dst, const rv<T, NS, vlayout::align>& src, int off) {
#pragma unroll
    for (int b = 0; b < NS / 32; ++b)
        if (lg() == 0) dst.data[off + 32 * b + lr()] = src.data[b][0];
    wave_fence();
}

// Products whose B operand stays in LDS: its fragments are read as the product consumes them instead of
// occupying a register tile (a 256x64 bf16 B would be 256 registers per lane).  The k <-> (lane half,
// slot) map is that of the register tiles: slot e of half h of lane half g is k = 16h + 8(e/4) + 4g + e%4.
// Fragments are requested `kStreamAhead` products ahead of their use (a small ring of registers) and the order is
// pinned with scheduling fences: left alone the compiler, at its register limit in these kernels, puts each read directly
// in front of its product and the wave sits out the LDS latency once per MFMA.
constexpr int kStreamAhead = 4;
// B as [N, K] rows (the DSL's mmaT): two 8-byte reads per fragment.
template <int M, int N, int K, int PAD>
__device__ __forceinline__ void mma_ABt(rt<float, M, N, layout::row>& d, const rt<bf16, M, K, layout::row>& a,
                                        const st<bf16, N, K, PAD>& b, const rt<float, M, N, layout::row>& c) {
    constexpr int KS = K / 16, NF = (N / 32) * KS, P = kStreamAhead;
    auto read = [&](int f) {
        const bf16* p = b.at(32 * (f / KS) + lr(), 16 * (f % KS) + 4 * lg());
        const bf16x4 lo = *reinterpret_cast<const bf16x4*>(p), hi = *reinterpret_cast<const bf16x4*>(p + 8);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    bf16x8 ring[P];
#pragma unroll
    for (int f = 0; f < P - 1 && f < NF; ++f) ring[f] = read(f);
    f32x16 acc[M / 32];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        const int nb = f / KS, ks = f % KS, kb = ks / 2, h = ks % 2;
        if (f + P - 1 < NF) ring[(f + P - 1) % P] = read(f + P - 1);
        __builtin_amdgcn_sched_barrier(0);
        if (ks == 0) {
#pragma unroll
            for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[mb][e] = c.data[mb][nb][e];
        }
#pragma unroll
        for (int mb = 0; mb < M / 32; ++mb) {
            bf16x8 fa;
#pragma unroll
            for (int e = 0; e < 8; ++e) fa[e] = a.data[mb][kb][8 * h + e];
            acc[mb] = mfma_32x32x16_bf16(ring[f % P], fa, acc[mb]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (ks == KS - 1) {
#pragma unroll
            for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
                for (int e = 0; e < 16; ++e) d.data[mb][nb][e] = acc[mb][e];
        }
    }
}
// E4M3 operands, B as [N, K] rows in LDS: a lane's 32 bytes of k for the 32x32x64 MFMA are the 16 bytes of its slots in two
// adjacent 32-column blocks (the map of the register tiles), i.e. eight 4-byte pieces at columns 32kb + 8q + 4g.
template <int M, int N, int K, int PAD>
__device__ __forceinline__ void mma_ABt(rt<float, M, N, layout::row>& d, const rt<fp8e4m3, M, K, layout::row>& a,
                                        const st<fp8e4m3, N, K, PAD>& b, const rt<float, M, N, layout::row>& c) {
    static_assert(K % 64 == 0, "E4M3 products consume k in steps of 64");
    constexpr int KS = K / 64, NF = (N / 32) * KS, P = 3;
    auto read = [&](int f) {
        i32x8 fb;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int wd = 0; wd < 4; ++wd)
                fb[4 * h + wd] = *reinterpret_cast<const int*>(b.at(32 * (f / KS) + lr(), 64 * (f % KS) + 32 * h + 8 * wd + 4 * lg()));
        return fb;
    };
    i32x8 ring[P];
#pragma unroll
    for (int f = 0; f < P - 1 && f < NF; ++f) ring[f] = read(f);
    f32x16 acc[M / 32];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        const int nb = f / KS, kb = 2 * (f % KS);
        if (f + P - 1 < NF) ring[(f + P - 1) % P] = read(f + P - 1);
        __builtin_amdgcn_sched_barrier(0);
        if (kb == 0) {
#pragma unroll
            for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[mb][e] = c.data[mb][nb][e];
        }
#pragma unroll
        for (int mb = 0; mb < M / 32; ++mb) {
            i32x8 fa;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int wd = 0; wd < 4; ++wd) {
                    uint32_t ua = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) ua |= (uint32_t)a.data[mb][kb + h][4 * wd + e].bits << (8 * e);
                    fa[4 * h + wd] = (int)ua;
                }
            acc[mb] = mfma_32x32x64_e4m3(ring[f % P], fa, acc[mb]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (kb == 2 * (KS - 1)) {
#pragma unroll
            for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
                for (int e = 0; e < 16; ++e) d.data[mb][nb][e] = acc[mb][e];
        }
    }
}
// B as [K, N] rows in LDS (the DSL's mma with a COL register tile): transposing reads, as load(rt col, st).
template <int M, int N, int K, int PAD>
__device__ __forceinline__ void mma_AB(rt<float, M, N, layout::row>& d, const rt<bf16, M, K, layout::row>& a,
                                       const st<bf16, K, N, PAD>& b, const rt<float, M, N, layout::row>& c) {
    const int i16 = lane() & 15, b16 = lane() >> 4;
    const int srow = 4 * (b16 >> 1) + (i16 >> 2), scol = 16 * (b16 & 1) + 4 * (i16 & 3);
    constexpr int KS = K / 16, NF = (N / 32) * KS, P = kStreamAhead;
    auto read = [&](int f) {
        const int nb = f / KS, ks = f % KS;
        const bf16x4 lo = ds_read_tr16(b.at(16 * ks + srow, 32 * nb + scol));
        const bf16x4 hi = ds_read_tr16(b.at(16 * ks + 8 + srow, 32 * nb + scol));
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    bf16x8 ring[P];
#pragma unroll
    for (int f = 0; f < P - 1 && f < NF; ++f) ring[f] = read(f);
    f32x16 acc[M / 32];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
        const int nb = f / KS, ks = f % KS, kb = ks / 2, h = ks % 2;
        if (f + P - 1 < NF) ring[(f + P - 1) % P] = read(f + P - 1);
        __builtin_amdgcn_sched_barrier(0);
        if (ks == 0) {
#pragma unroll
            for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[mb][e] = c.data[mb][nb][e];
        }
#pragma unroll
        for (int mb = 0; mb < M / 32; ++mb) {
            bf16x8 fa;
#pragma unroll
            for (int e = 0; e < 8; ++e) fa[e] = a.data[mb][kb][8 * h + e];
            acc[mb] = mfma_32x32x16_bf16(ring[f % P], fa, acc[mb]);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (ks == KS - 1) {
#pragma unroll
            for (int mb = 0; mb < M / 32; ++mb)
#pragma unroll
                for (int e = 0; e < 16; ++e) d.data[mb][nb][e] = acc[mb][e];
        }
    }
}

}  // namespace wave
}  // namespace tile
}  // namespace tyr
