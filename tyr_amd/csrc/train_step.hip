// The element-wise half of the reference's attention train step (gfx950), fused into two streaming kernels.
//
// Reference semantics (Examples/GPU/RunMhaH100Train.lean:60-93, `oneKernelTrainStep`), which the reference
// evaluates as a chain of LibTorch element-wise calls around its forward and backward kernels:
//   lossAndGradOut  :60-67   diff = f32(out) - f32(target);  loss = 0.5 * mean(diff * diff);
//                            dO = bf16(diff / nElems)
//   sgdUpdate       :69-70   param' = param - (grad * lr)            (f32 master, grad = f32(bf16 gradient))
//   :83-85                   q = bf16(qM) ... at the top of the next step
// Here: one pass over out / target writes dO and per-workgroup partial sums of diff^2 (a second, single
// workgroup turns them into the loss); one pass per parameter reads the f32 master and the bf16 gradient and
// writes the updated master together with its bf16 copy for the next step's kernels.  Both are bound by HBM
// bandwidth: 16-byte pieces per lane, consecutive lanes on consecutive addresses, non-temporal hints, no loop.
// Products and differences are evaluated as separate f32 operations (no fused multiply-add) and the division
// is a true division, so dO and the updated masters are bit-identical to the LibTorch chain.
#include "../../include/tyr_hip.h"

#include <limits.h>

#include "common.hpp"

namespace tyr {
namespace {

constexpr int THREADS = 256;

__device__ __forceinline__ void unpack8(u32x4 v, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[2 * i] = bf16_lo(v[i]); f[2 * i + 1] = bf16_hi(v[i]); }
}

// one 8-element piece per lane; partial[blockIdx.x] = sum over the workgroup of diff^2
__global__ __launch_bounds__(THREADS) void mse_grad_kernel(const uint16_t* __restrict__ out, const uint16_t* __restrict__ target,
                                                           uint16_t* __restrict__ d_out, float* __restrict__ partial,
                                                           size_t pieces, float n_elems) {
    __shared__ float wave_sum[THREADS / 64];
    const size_t i = (size_t)blockIdx.x * THREADS + threadIdx.x;
    float acc = 0.0f;
    if (i < pieces) {
        float o[8], t[8], d[8];
        unpack8(ld_global_16_nt(out + 8 * i), o);
        unpack8(ld_global_16_nt(target + 8 * i), t);
        u32x4 g;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
#pragma clang fp contract(off)
            d[e] = o[e] - t[e];
            acc = acc + d[e] * d[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) g[e] = pack_bf16(d[2 * e] / n_elems, d[2 * e + 1] / n_elems);
        st_global_16_nt(d_out + 8 * i, g);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
}

// loss = 0.5 * (sum of the partials) / n, summed in double by one workgroup
__global__ __launch_bounds__(1024) void mse_loss_kernel(const float* __restrict__ partial, size_t count, double n_elems,
                                                        float* __restrict__ loss) {
    __shared__ double part[16];
    double acc = 0.0;
    for (size_t i = threadIdx.x; i < count; i += 1024) acc += (double)partial[i];
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = 0.0;
        for (int w = 0; w < 16; ++w) s += part[w];
        *loss = (float)(0.5 * s / n_elems);
    }
}

// param' = param - (f32(grad) * lr); optionally also bf16(param').  param_out may be param itself (the in-place update), so
// neither of the two is declared restrict; a lane stores only the elements it loaded.
__global__ __launch_bounds__(THREADS) void sgd_kernel(const float* param, const uint16_t* __restrict__ grad, float lr,
                                                      float* param_out, uint16_t* __restrict__ param_out_bf16,
                                                      size_t pieces) {
    const size_t i = (size_t)blockIdx.x * THREADS + threadIdx.x;
    if (i >= pieces) return;
    const f32x4 p0 = __builtin_bit_cast(f32x4, ld_global_16_nt(param + 8 * i));
    const f32x4 p1 = __builtin_bit_cast(f32x4, ld_global_16_nt(param + 8 * i + 4));
    float g[8], r[8];
    unpack8(ld_global_16_nt(grad + 8 * i), g);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
#pragma clang fp contract(off)
        const float step = g[e] * lr;
        r[e] = (e < 4 ? p0[e] : p1[e - 4]) - step;
    }
    st_global_16_nt(param_out + 8 * i, __builtin_bit_cast(u32x4, f32x4{r[0], r[1], r[2], r[3]}));
    st_global_16_nt(param_out + 8 * i + 4, __builtin_bit_cast(u32x4, f32x4{r[4], r[5], r[6], r[7]}));
    if (param_out_bf16 != nullptr) {
        u32x4 b;
#pragma unroll
        for (int e = 0; e < 4; ++e) b[e] = pack_bf16(r[2 * e], r[2 * e + 1]);
        st_global_16_nt(param_out_bf16 + 8 * i, b);
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace
}  // namespace tyr

extern "C" {

size_t tyr_hip_mse_loss_grad_workspace_bytes(uint64_t n) {
    const uint64_t pieces = (n + 7) / 8;
    return (size_t)((pieces + tyr::THREADS - 1) / tyr::THREADS) * sizeof(float);
}

int tyr_hip_mse_loss_grad(const void* out, const void* target, void* d_out, float* loss, uint64_t n, void* workspace,
                          size_t workspace_bytes, void* stream) {
    using namespace tyr;
    if (!out || !target || !d_out || !loss) return TYR_HIP_ERR_NULL_POINTER;
    if (n == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (n % 8 != 0) return TYR_HIP_ERR_UNSUPPORTED;
    const uint64_t pieces = n / 8, blocks = (pieces + THREADS - 1) / THREADS;
    if (blocks > (uint64_t)INT_MAX) return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(out) || !aligned16(target) || !aligned16(d_out) || (reinterpret_cast<uintptr_t>(loss) & 3u))
        return TYR_HIP_ERR_MISALIGNED;
    if (!workspace || workspace_bytes < tyr_hip_mse_loss_grad_workspace_bytes(n)) return TYR_HIP_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) & 3u) return TYR_HIP_ERR_MISALIGNED;
    auto s = static_cast<hipStream_t>(stream);
    float* partial = static_cast<float*>(workspace);
    hipLaunchKernelGGL(mse_grad_kernel, dim3((unsigned)blocks), dim3(THREADS), 0, s, static_cast<const uint16_t*>(out),
                       static_cast<const uint16_t*>(target), static_cast<uint16_t*>(d_out), partial, (size_t)pieces, (float)n);
    if (hipGetLastError() != hipSuccess) return TYR_HIP_ERR_LAUNCH;
    hipLaunchKernelGGL(mse_loss_kernel, dim3(1), dim3(1024), 0, s, partial, (size_t)blocks, (double)n, loss);
    return hipGetLastError() == hipSuccess ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_sgd_step(const float* param, const void* grad, float lr, float* param_out, void* param_out_bf16, uint64_t n,
                     void* stream) {
    using namespace tyr;
    if (!param || !grad || !param_out) return TYR_HIP_ERR_NULL_POINTER;
    if (n == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (n % 8 != 0) return TYR_HIP_ERR_UNSUPPORTED;
    const uint64_t pieces = n / 8, blocks = (pieces + THREADS - 1) / THREADS;
    if (blocks > (uint64_t)INT_MAX) return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(param) || !aligned16(grad) || !aligned16(param_out) || !aligned16(param_out_bf16))
        return TYR_HIP_ERR_MISALIGNED;
    hipLaunchKernelGGL(sgd_kernel, dim3((unsigned)blocks), dim3(THREADS), 0, static_cast<hipStream_t>(stream), param,
                       static_cast<const uint16_t*>(grad), lr, param_out, static_cast<uint16_t*>(param_out_bf16), (size_t)pieces);
    return hipGetLastError() == hipSuccess ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

}  // extern "C"
