// Memory-bound row kernels around the attention path (gfx950): device copy, rotary embedding,
// fused residual + LayerNorm, and the decode step's "rotate q and k, append k and v to the cache".
//
// Reference semantics restated here:
//   copy           Tyr/GPU/Kernels/Copy.lean:16-27 (copy64x64: out = in, one f32 tile per block)
//   rotary         cc/src/tyr.cpp:3837-3873 (lean_torch_apply_rotary_emb): x = [x1 | x2] split in
//                  halves along head_dim, y1 = x1 cos - x2 sin, y2 = x1 sin + x2 cos, cos / sin
//                  [seq, head_dim/2] f32 broadcast over batch and heads, arithmetic in f32, result in
//                  x's dtype; DSL twin Tyr/GPU/Kernels/Rotary.lean:13-66 (rotaryFwd, f32 64x64).
//   layernorm      Tyr/GPU/Kernels/FusedLayerNorm.lean:28-140 (tkFusedLayerNormResidual1024):
//                  out_resid = bf16(x + residual); statistics of the rounded out_resid in f32 over the
//                  whole row; out = bf16((r - mean) * rsqrt(var + eps) * weight + bias); expected
//                  values Examples/GPU/RunLayerNorm.lean:27-33 (torch layer_norm of x + residual).
//   decode append  Tyr/Model/Qwen/Attention.lean:172-196 (forwardStep): applyRotaryEmb on the
//                  single-token q and k, then sliceScatter of k and v into row `seq` of the
//                  [batch, kv_heads, maxLen, head_dim] cache.
//
// All four are bound by HBM bandwidth: every lane moves 16-byte pieces, consecutive lanes touch
// consecutive addresses, and the grids have many more workgroups than the device has CUs.
#include "common.hpp"
#include "launch.hpp"

namespace tyr {

namespace rw {
constexpr int THREADS = 256;
constexpr int STREAM_THREADS = 64;      // one wave per workgroup for the pure streaming kernels

__device__ __forceinline__ void unpack8(u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[2 * i] = bf16_lo(v[i]); f[2 * i + 1] = bf16_hi(v[i]); }
}
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = pack_bf16(f[2 * i], f[2 * i + 1]);
    return v;
}

// Rotates one 16-byte piece pair: a = elements [e0, e0+E) of the first half, b = the same
// elements of the second half; c / s point at cos[e0], sin[e0].
template <typename T> struct Piece;
template <> struct Piece<float> {
    static constexpr int E = 4;
    static __device__ __forceinline__ void rotate(u32x4& a, u32x4& b, const float* c, const float* s) {
        const f32x4 cv = *reinterpret_cast<const f32x4*>(c), sv = *reinterpret_cast<const f32x4*>(s);
        f32x4 x1 = __builtin_bit_cast(f32x4, a), x2 = __builtin_bit_cast(f32x4, b), y1, y2;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma clang fp contract(off)   // separate multiplies and add, as the reference expression evaluates
            y1[i] = x1[i] * cv[i] - x2[i] * sv[i];
            y2[i] = x1[i] * sv[i] + x2[i] * cv[i];
        }
        a = __builtin_bit_cast(u32x4, y1);
        b = __builtin_bit_cast(u32x4, y2);
    }
};
template <> struct Piece<uint16_t> {                 // bf16
    static constexpr int E = 8;
    static __device__ __forceinline__ void rotate(u32x4& a, u32x4& b, const float* c, const float* s) {
        float x1[8], x2[8], y1[8], y2[8], cv[8], sv[8];
        unpack8(a, x1);
        unpack8(b, x2);
        *reinterpret_cast<f32x4*>(cv) = *reinterpret_cast<const f32x4*>(c);
        *reinterpret_cast<f32x4*>(cv + 4) = *reinterpret_cast<const f32x4*>(c + 4);
        *reinterpret_cast<f32x4*>(sv) = *reinterpret_cast<const f32x4*>(s);
        *reinterpret_cast<f32x4*>(sv + 4) = *reinterpret_cast<const f32x4*>(s + 4);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma clang fp contract(off)
            y1[i] = x1[i] * cv[i] - x2[i] * sv[i];
            y2[i] = x1[i] * sv[i] + x2[i] * cv[i];
        }
        a = pack8(y1);
        b = pack8(y2);
    }
};
}  // namespace rw

// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(rw::THREADS) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                           size_t n16, const unsigned char* __restrict__ src_tail,
                                                           unsigned char* __restrict__ dst_tail, int tail) {
    // One 16-byte piece per lane, one wave per workgroup, no loop: the dispatcher then walks the
    // buffers as one contiguous front (measured on a 1 GiB copy: 6.7 TB/s of read + write traffic,
    // against 6.0 for a grid-stride loop with four loads in flight per lane).
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n16) st_global_16_nt(dst + i, ld_global_16_nt(src + i));
    if (blockIdx.x == 0 && (int)threadIdx.x < tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];
}

// x, y: [rows_total = B*S*H][D]; row -> position s = (row / H) % S.  One thread rotates one piece
// pair; a row takes D / (2E) consecutive threads.
template <typename T>
__global__ __launch_bounds__(rw::THREADS) void rope_kernel(const T* __restrict__ x, const float* __restrict__ cosp,
                                                           const float* __restrict__ sinp, T* __restrict__ y,
                                                           size_t rows, int S, int H, int D) {
    constexpr int E = rw::Piece<T>::E;
    const int per_row = D / (2 * E);
    const size_t id = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t row = id / per_row;
    if (row >= rows) return;
    const int e0 = (int)(id % per_row) * E;
    const int s = (int)((row / H) % S);
    const T* xr = x + row * D;
    u32x4 a = ld_global_16_nt(xr + e0), b = ld_global_16_nt(xr + D / 2 + e0);
    rw::Piece<T>::rotate(a, b, cosp + (size_t)s * (D / 2) + e0, sinp + (size_t)s * (D / 2) + e0);
    T* yr = y + row * D;
    st_global_16_nt(yr + e0, a);
    st_global_16_nt(yr + D / 2 + e0, b);
}

// Rows 0 .. B*Hq-1: q rows (rotated into q_out).  Then B*Hkv k rows (rotated into row `pos` of the
// k cache) and B*Hkv v rows (copied into row `pos` of the v cache).  cos / sin: [D/2] of position pos.
__global__ __launch_bounds__(rw::THREADS) void decode_rope_append_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k_new, const uint16_t* __restrict__ v_new,
    const float* __restrict__ cosp, const float* __restrict__ sinp, uint16_t* __restrict__ q_out,
    uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache, int nq, int nkv, int D, size_t kv_stride,
    size_t pos) {
    const int per_row = D / 16;
    const int id = blockIdx.x * blockDim.x + threadIdx.x;
    const int row = id / per_row;
    if (row >= nq + 2 * nkv) return;
    const int e0 = (id % per_row) * 8;
    const uint16_t* src;
    uint16_t* dst;
    bool rotate = true;
    if (row < nq) {
        src = q + (size_t)row * D;
        dst = q_out + (size_t)row * D;
    } else if (row < nq + nkv) {
        src = k_new + (size_t)(row - nq) * D;
        dst = k_cache + ((size_t)(row - nq) * kv_stride + pos) * D;
    } else {
        src = v_new + (size_t)(row - nq - nkv) * D;
        dst = v_cache + ((size_t)(row - nq - nkv) * kv_stride + pos) * D;
        rotate = false;
    }
    u32x4 a = ld_global_16(src + e0), b = ld_global_16(src + D / 2 + e0);
    if (rotate) rw::Piece<uint16_t>::rotate(a, b, cosp + e0, sinp + e0);
    st_global_16(dst + e0, a);
    st_global_16(dst + D / 2 + e0, b);
}

// One wave per row; a lane holds pieces lane, lane + 64, ... of the row (8 bf16 each).
template <int MAXP>
__global__ __launch_bounds__(rw::THREADS) void layernorm_residual_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ res, const uint16_t* __restrict__ weight,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ out, uint16_t* __restrict__ out_resid, size_t rows,
    int d_model, float eps) {
    const int lane = threadIdx.x & 63;
    const size_t row = (size_t)blockIdx.x * (rw::THREADS / 64) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int pieces = d_model / 8;
    const uint16_t* xr = x + row * d_model;
    const uint16_t* rr = res + row * d_model;
    float v[MAXP][8];
    float sum = 0.0f;
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {
        const int pc = lane + 64 * p;
        if (pc < pieces) {
            float a[8], b[8];
            rw::unpack8(ld_global_16_nt(xr + pc * 8), a);
            rw::unpack8(ld_global_16_nt(rr + pc * 8), b);
#pragma unroll
            for (int i = 0; i < 8; ++i) a[i] += b[i];
            const u32x4 r16 = rw::pack8(a);                     // out_resid is the bf16-rounded sum ...
            st_global_16_nt(out_resid + row * d_model + pc * 8, r16);
            rw::unpack8(r16, v[p]);                             // ... and the statistics are taken from it
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += v[p][i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[p][i] = 0.0f;
        }
    }
    auto wave_sum = [](float s) {
#pragma unroll
        for (int o = 1; o < 32; o <<= 1) s += __shfl_xor(s, o, 64);
        return sum_xor32(s);
    };
    const float mean = wave_sum(sum) / (float)d_model;
    float sq = 0.0f;
#pragma unroll
    for (int p = 0; p < MAXP; ++p)
        if (lane + 64 * p < pieces) {
#pragma unroll
            for (int i = 0; i < 8; ++i) { const float c = v[p][i] - mean; sq += c * c; }
        }
    const float inv_std = rsqrtf(wave_sum(sq) / (float)d_model + eps);
#pragma unroll
    for (int p = 0; p < MAXP; ++p) {
        const int pc = lane + 64 * p;
        if (pc < pieces) {
            float w[8], b[8], o[8];
            rw::unpack8(ld_global_16(weight + pc * 8), w);
            rw::unpack8(ld_global_16(bias + pc * 8), b);
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = (v[p][i] - mean) * inv_std * w[i] + b[i];
            st_global_16_nt(out + row * d_model + pc * 8, rw::pack8(o));
        }
    }
}

// ------------------------------------------------------------------------------------------
int launch_copy(const void* src, void* dst, size_t bytes, hipStream_t stream) {
    const size_t n16 = bytes / 16;
    const int tail = (int)(bytes % 16);
    size_t blocks = (n16 + rw::STREAM_THREADS - 1) / rw::STREAM_THREADS;
    if (blocks == 0) blocks = 1;
    if (blocks > 0x7fffffffull) return -1;             // 2^31 workgroups of 1 KiB: 2 TiB
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(rw::STREAM_THREADS), 0, stream,
                       static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), n16,
                       static_cast<const unsigned char*>(src) + n16 * 16, static_cast<unsigned char*>(dst) + n16 * 16,
                       tail);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_rope_fwd(const void* x, const float* cosp, const float* sinp, void* y, size_t rows, int S, int H, int D,
                    int is_bf16, hipStream_t stream) {
    const size_t threads = rows * (size_t)(D / (is_bf16 ? 16 : 8));
    const size_t blocks = (threads + rw::THREADS - 1) / rw::THREADS;
    if (is_bf16)
        hipLaunchKernelGGL(rope_kernel<uint16_t>, dim3((unsigned)blocks), dim3(rw::THREADS), 0, stream,
                           static_cast<const uint16_t*>(x), cosp, sinp, static_cast<uint16_t*>(y), rows, S, H, D);
    else
        hipLaunchKernelGGL(rope_kernel<float>, dim3((unsigned)blocks), dim3(rw::THREADS), 0, stream,
                           static_cast<const float*>(x), cosp, sinp, static_cast<float*>(y), rows, S, H, D);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_decode_rope_append(const void* q, const void* k_new, const void* v_new, const float* cosp,
                              const float* sinp, void* q_out, void* k_cache, void* v_cache, int B, int Hq, int Hkv,
                              int D, size_t kv_stride, size_t pos, hipStream_t stream) {
    const int nq = B * Hq, nkv = B * Hkv;
    const size_t threads = (size_t)(nq + 2 * nkv) * (D / 16);
    const size_t blocks = (threads + rw::THREADS - 1) / rw::THREADS;
    hipLaunchKernelGGL(decode_rope_append_kernel, dim3((unsigned)blocks), dim3(rw::THREADS), 0, stream,
                       static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k_new),
                       static_cast<const uint16_t*>(v_new), cosp, sinp, static_cast<uint16_t*>(q_out),
                       static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), nq, nkv, D, kv_stride, pos);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

int launch_layernorm_residual(const void* x, const void* residual, const void* weight, const void* bias, void* out,
                              void* out_resid, size_t rows, int d_model, float eps, hipStream_t stream) {
    const size_t blocks = (rows + 3) / 4;
    const int pieces_per_lane = (d_model / 8 + 63) / 64;
#define TYR_LN_LAUNCH(MAXP)                                                                                     \
    hipLaunchKernelGGL(layernorm_residual_kernel<MAXP>, dim3((unsigned)blocks), dim3(rw::THREADS), 0, stream,   \
                       static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(residual),                 \
                       static_cast<const uint16_t*>(weight), static_cast<const uint16_t*>(bias),                \
                       static_cast<uint16_t*>(out), static_cast<uint16_t*>(out_resid), rows, d_model, eps)
    if (pieces_per_lane <= 2) TYR_LN_LAUNCH(2);
    else if (pieces_per_lane <= 4) TYR_LN_LAUNCH(4);
    else if (pieces_per_lane <= 8) TYR_LN_LAUNCH(8);
    else TYR_LN_LAUNCH(16);
#undef TYR_LN_LAUNCH
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

}  // namespace tyr
