// Calibration kernels: what the matrix cores of this device sustain on given operand bits.
//
// A wave loads NF row fragments and NF column fragments from the caller's buffer once, then issues
// nothing but MFMAs: `iters` rounds of NF x NF products, round-robin over four independent
// accumulators, every product on a different pair of operand registers.  No LDS, no memory
// traffic, no vector instruction in the loop.  The rate this reaches with normally distributed
// operands is the ceiling any kernel built on the same MFMA can approach on this device with such
// data (the clock the device holds under matrix load depends on the bits that toggle in the operand
// paths), and is what bench.py reports as `roofline.sustained_peak` beside the nominal peak.
#include "../../include/tyr_hip.h"

#include <hip/hip_runtime.h>

#include "common.hpp"

namespace tyr {
namespace {

constexpr int NF = 4;   // fragments per operand side held in registers

// DT = 0: 32x32x16 bf16 (16 B per lane per fragment).  DT = 1: 32x32x64 E4M3 (32 B per lane).
template <int DT>
__global__ __launch_bounds__(256) void mfma_sustain_kernel(const unsigned char* __restrict__ operands,
                                                           size_t operand_bytes, int iters,
                                                           float* __restrict__ sink) {
    constexpr int FB = DT == 0 ? 16 : 32;                    // bytes per lane per fragment
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    // every wave reads its own 2 * NF * 64 * FB bytes (wrapping inside the buffer)
    const size_t span = (size_t)2 * NF * 64 * FB;
    const size_t nspans = operand_bytes / span;              // >= 1, checked by the host
    const unsigned char* base = operands + (wave % nspans) * span + (size_t)lane * FB;

    f32x16 acc[4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[a][e] = 0.0f;

    if constexpr (DT == 0) {
        bf16x8 ra[NF], rb[NF];
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            ra[i] = __builtin_bit_cast(bf16x8, ld_global_16(base + (size_t)i * 64 * FB));
            rb[i] = __builtin_bit_cast(bf16x8, ld_global_16(base + (size_t)(NF + i) * 64 * FB));
        }
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < NF; ++i)
#pragma unroll
                for (int j = 0; j < NF; ++j)
                    acc[(i * NF + j) & 3] = mfma_32x32x16_bf16(ra[i], rb[(i + j) % NF], acc[(i * NF + j) & 3]);
        }
    } else {
        i32x8 ra[NF], rb[NF];
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            const u32x4 a0 = ld_global_16(base + (size_t)i * 64 * FB), a1 = ld_global_16(base + (size_t)i * 64 * FB + 16);
            const u32x4 b0 = ld_global_16(base + (size_t)(NF + i) * 64 * FB),
                        b1 = ld_global_16(base + (size_t)(NF + i) * 64 * FB + 16);
            ra[i] = i32x8{(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
            rb[i] = i32x8{(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
        }
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < NF; ++i)
#pragma unroll
                for (int j = 0; j < NF; ++j)
                    acc[(i * NF + j) & 3] = mfma_32x32x64_e4m3(ra[i], rb[(i + j) % NF], acc[(i * NF + j) & 3]);
        }
    }

    // one value per lane keeps the products alive; 64 floats per wave
    float s = 0.0f;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[a][e];
    sink[wave * 64 + lane] = s;
}

}  // namespace
}  // namespace tyr

extern "C" int tyr_hip_mfma_sustain(const void* operands, size_t operand_bytes, int dtype, uint64_t workgroups,
                                    uint64_t iters, float* sink, size_t sink_bytes, double* flop_per_launch, void* stream) {
    using namespace tyr;
    if (!operands || !sink) return TYR_HIP_ERR_NULL_POINTER;
    if (workgroups <= (1u << 24) && sink_bytes < (size_t)workgroups * 256 * sizeof(float)) return TYR_HIP_ERR_WORKSPACE;
    if (dtype != TYR_HIP_MFMA_BF16 && dtype != TYR_HIP_MFMA_E4M3) return TYR_HIP_ERR_UNSUPPORTED;
    const size_t span = (size_t)2 * NF * 64 * (dtype == TYR_HIP_MFMA_BF16 ? 16 : 32);
    if (workgroups == 0 || iters == 0 || workgroups > (1u << 24) || iters > (1u << 30) || operand_bytes < span)
        return TYR_HIP_ERR_BAD_SHAPE;
    if (reinterpret_cast<uintptr_t>(operands) & 15u) return TYR_HIP_ERR_MISALIGNED;
    const double k = dtype == TYR_HIP_MFMA_BF16 ? 16.0 : 64.0;
    if (flop_per_launch) *flop_per_launch = 2.0 * 32 * 32 * k * NF * NF * (double)iters * 4.0 * (double)workgroups;
    auto ops = static_cast<const unsigned char*>(operands);
    if (dtype == TYR_HIP_MFMA_BF16)
        hipLaunchKernelGGL(mfma_sustain_kernel<0>, dim3((unsigned)workgroups), dim3(256), 0,
                           static_cast<hipStream_t>(stream), ops, operand_bytes, (int)iters, sink);
    else
        hipLaunchKernelGGL(mfma_sustain_kernel<1>, dim3((unsigned)workgroups), dim3(256), 0,
                           static_cast<hipStream_t>(stream), ops, operand_bytes, (int)iters, sink);
    return hipGetLastError() == hipSuccess ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}
