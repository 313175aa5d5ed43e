// Shared device-side vocabulary for the gfx950 kernels: vector types, MFMA wrappers,
// bf16 packing, cross-lane helpers.  Wave size is 64 everywhere.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tyr {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;

constexpr int kWave = 64;

// ---- MFMA (dense, f32 accumulate) -------------------------------------------------
// Operand layout facts used throughout (lane = l, wave64):
//   32x32x16 bf16 : A lane holds row  l%32, k = 8*(l/32)+[0,8) ; B lane holds col l%32, same k.
//                   D reg r (0..15)  <-> row 8*(r/4) + 4*(l/32) + r%4, col l%32.
//   16x16x32 bf16 : A lane holds row  l%16, k = 8*(l/16)+[0,8) ; B lane holds col l%16, same k.
//                   D reg r (0..3)   <-> row 4*(l/16) + r, col l%16.
//   32x32x64 fp8  : as 32x32x16 with 32 bytes of k per lane (k = 32*(l/32)+[0,32)).
// Only "A and B use the same k <-> (lane group, slot) map" matters for correctness of a
// product, so kernels are free to permute k as long as both operands agree.

__device__ __forceinline__ f32x16 mfma_32x32x16_bf16(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma_16x16x32_bf16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// FP8 E4M3 x E4M3 (format code 0 on both operands), scales fixed at 1 (unscaled encoding).
__device__ __forceinline__ f32x16 mfma_32x32x64_e4m3(i32x8 a, i32x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

// ---- bf16 packing -----------------------------------------------------------------
// Round-to-nearest-even f32 -> bf16 pair (v_cvt_pk_bf16_f32); lo goes to bits [15:0].
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    bf16x2 r = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __builtin_bit_cast(float, u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __builtin_bit_cast(float, u & 0xffff0000u); }

// ---- cross-lane -------------------------------------------------------------------
// Value held by lane l^32.  v_permlane32_swap exchanges lanes 32-63 of its first register with
// lanes 0-31 of its second; fed the same value twice, the partner's value is in the first
// result for the upper half-wave and in the second for the lower half-wave.  (Selecting per
// half also stays right if the compiler assigns both operands to one register, in which case
// either result holds the partner's value.)
__device__ __forceinline__ float xor32(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    u32x2 s = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    uint32_t other = (threadIdx.x & 32) ? s.x : s.y;
    return __builtin_bit_cast(float, other);
}
// Value held by lane l^16 (same construction with v_permlane16_swap on 16-lane rows).
__device__ __forceinline__ float xor16(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    u32x2 s = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    uint32_t other = (threadIdx.x & 16) ? s.x : s.y;
    return __builtin_bit_cast(float, other);
}
__device__ __forceinline__ float max_xor32(float x) { return fmaxf(x, xor32(x)); }
__device__ __forceinline__ float sum_xor32(float x) { return x + xor32(x); }
__device__ __forceinline__ float max_xor16(float x) { return fmaxf(x, xor16(x)); }
__device__ __forceinline__ float sum_xor16(float x) { return x + xor16(x); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- 16-byte global / LDS moves ----------------------------------------------------
__device__ __forceinline__ u32x4 ld_global_16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ u32x2 ld_global_8(const void* p) { return *reinterpret_cast<const u32x2*>(p); }
__device__ __forceinline__ void st_global_16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
// Streaming variants (non-temporal hint) for data that is touched once: the lines are not kept in
// the caches at the expense of reusable data.  On the decode and copy kernels this alone is worth
// 10-30 % of the achieved HBM bandwidth.
__device__ __forceinline__ u32x4 ld_global_16_nt(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void st_global_16_nt(void* p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}
__device__ __forceinline__ void st_global_8(void* p, u32x2 v) { *reinterpret_cast<u32x2*>(p) = v; }

// 8x8 transpose of 16-bit elements held as 8 rows of 4 dwords: out[c] holds column c
// (8 elements = 4 dwords, element r in half (r&1) of dword r/2).
__device__ __forceinline__ void transpose8x8_b16(const u32x4 (&in)[8], u32x4 (&out)[8]) {
#pragma unroll
    for (int c2 = 0; c2 < 4; ++c2) {      // column pair (2*c2, 2*c2+1) lives in dword c2 of every row
        u32x4 lo, hi;
#pragma unroll
        for (int j = 0; j < 4; ++j) {     // output dword j packs rows 2j, 2j+1
            uint32_t x0 = in[2 * j][c2], x1 = in[2 * j + 1][c2];
            lo[j] = __builtin_amdgcn_perm(x1, x0, 0x05040100u);   // [x0.lo16, x1.lo16]
            hi[j] = __builtin_amdgcn_perm(x1, x0, 0x07060302u);   // [x0.hi16, x1.hi16]
        }
        out[2 * c2] = lo;
        out[2 * c2 + 1] = hi;
    }
}

// Makes the compiler treat v as produced here: any load feeding it is waited for at this point
// (and not, conservatively, at its first use inside a loop that has other loads in flight).
__device__ __forceinline__ void pin_registers(bf16x8& v) {
    u32x4 u = __builtin_bit_cast(u32x4, v);
    asm volatile("" : "+v"(u));
    v = __builtin_bit_cast(bf16x8, u);
}

// ds_read_b64_tr_b8: transposing LDS read for bytes.  Within each block of 16 lanes, lane 8q+p
// receives byte p of the 8-byte pieces addressed by lanes q, q+2, q+4, ..., q+14 of the block.
__device__ __forceinline__ u32x2 ds_read_tr8(const void* lds_ptr) {
    typedef __attribute__((ext_vector_type(2))) int i32x2;
    const i32x2 v = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2*)(lds_ptr));
    return __builtin_bit_cast(u32x2, v);
}

// Buffer resource (V#) for raw byte-addressed access to [base, base + bytes): loads beyond the
// range return zero.  On gfx950 the range check covers the whole offset, per-lane, scalar and immediate
// parts together (probed with a 4 KiB descriptor inside a larger allocation: a scalar offset of 4000
// gives data to the lanes below byte 4096 and zeros to the rest), so a slice index carried in the
// scalar offset is zero-filled past the end like a row index carried in the per-lane offset.
__device__ __forceinline__ u32x4 make_raw_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    return u32x4{(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
}

// 16 bytes per lane from global memory straight into LDS: lane i of the wave writes
// lds_base + 16 i (lds_base wave-uniform); the source is rsrc.base + voffset + soffset.
// Issued as opaque asm so that the compiler does not order later LDS reads behind it; the
// caller waits with wait_vmcnt0() (and a barrier) before anyone reads the destination.  M0 is
// written here.  M0 is a reserved register for this compiler (it never holds a value across
// statements; the compiler writes it right before each of its own instructions that read it, and
// hipcc rejects it on a clobber list with a warning), so the write cannot corrupt compiler state as
// long as no compiler-generated M0 reader sits between its own write and use -- which
// tests/test_m0_discipline.py checks on the assembly of every kernel file that includes this one:
// the only M0 accesses are these writes, each followed by the LDS-DMA loads that consume it.
__device__ __forceinline__ void load_global_to_lds_16(u32x4 rsrc, uint32_t lds_base, int voffset, int soffset) {
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "buffer_load_dwordx4 %1, %2, %3 offen lds"
        :
        : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
        : "memory");
}
// N consecutive kilobytes of LDS from one M0 write: the instruction's immediate offset advances the
// LDS destination and the global source together, so request m uses immediate 1024 m and a per-lane
// offset that has 1024 m taken off (voffset_less[m] = source offset of request m - 1024 m >= 0).
template <int N>
__device__ __forceinline__ void load_global_to_lds_16xN(u32x4 rsrc, uint32_t lds_base, const int (&voffset_less)[N], int soffset) {
    static_assert(N == 1 || N == 2 || N == 4, "1, 2 or 4 requests per call");
    if constexpr (N == 1) {
        load_global_to_lds_16(rsrc, lds_base, voffset_less[0], soffset);
    } else if constexpr (N == 4) {
        asm volatile(
            "s_mov_b32 m0, %0\n\t"
            "s_nop 0\n\t"
            "buffer_load_dwordx4 %1, %5, %6 offen lds\n\t"
            "buffer_load_dwordx4 %2, %5, %6 offen offset:1024 lds\n\t"
            "buffer_load_dwordx4 %3, %5, %6 offen offset:2048 lds\n\t"
            "buffer_load_dwordx4 %4, %5, %6 offen offset:3072 lds"
            :
            : "s"(lds_base), "v"(voffset_less[0]), "v"(voffset_less[1]), "v"(voffset_less[2]), "v"(voffset_less[3]),
              "s"(rsrc), "s"(soffset)
            : "memory");
    } else {
        asm volatile(
            "s_mov_b32 m0, %0\n\t"
            "s_nop 0\n\t"
            "buffer_load_dwordx4 %1, %3, %4 offen lds\n\t"
            "buffer_load_dwordx4 %2, %3, %4 offen offset:1024 lds"
            :
            : "s"(lds_base), "v"(voffset_less[0]), "v"(voffset_less[1]), "s"(rsrc), "s"(soffset)
            : "memory");
    }
}
__device__ __forceinline__ void wait_vmcnt0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ds_read_b64_tr_b16: transposing LDS read.  Within each block of 16 lanes, lane 4q+p receives
// element p (16 bits) of the 8-byte pieces addressed by lanes q, q+4, q+8, q+12 of the block.
__device__ __forceinline__ bf16x4 ds_read_tr16(const void* lds_ptr) {
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(lds_ptr));
    return __builtin_bit_cast(bf16x4, v);
}

// Epilogue of the 256x256-tile GEMMs: one wave's 128x128 f32 accumulator quadrant (4x4 MFMA tiles
// computed with the B fragment as row operand: lane = m row l%32, register e <-> n = 8(e/4) +
// 4(l/32) + e%4) goes to global memory as bf16 rows.  Each 32-row band passes through a private
// LDS scratch (32 rows x 272 B) so that the global stores are 16 bytes per lane along rows.
constexpr int kEpilogueScratchBytes = 32 * 272;
// rows / cols = how much of the 128x128 quadrant lies inside C (cols a multiple of 8).
// NJ = 32-column tiles of the wave's block (4: a 128x128 quadrant; 2: 128x64).
template <int NJ>
__device__ __forceinline__ void store_quadrant_bf16(const f32x16 (&acc)[4][NJ], float scale, unsigned char* scratch,
                                                    uint16_t* c_quadrant, int ldc, int lane, int rows, int cols) {
    const int r = lane & 31, g = lane >> 5;
    constexpr int CH = NJ * 4;                           // 16-byte chunks per row of the block
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                u32x2 v;
                v.x = pack_bf16(acc[i][j][q4 * 4 + 0] * scale, acc[i][j][q4 * 4 + 1] * scale);
                v.y = pack_bf16(acc[i][j][q4 * 4 + 2] * scale, acc[i][j][q4 * 4 + 3] * scale);
                *reinterpret_cast<u32x2*>(scratch + r * 272 + (j * 32 + q4 * 8 + g * 4) * 2) = v;
            }
#pragma unroll
        for (int k = 0; k < 32 * CH / 64; ++k) {
            const int row = lane / CH + (64 / CH) * k;
            const u32x4 v = *reinterpret_cast<const u32x4*>(scratch + row * 272 + (lane % CH) * 16);
            if (i * 32 + row < rows && (lane % CH) * 8 < cols)
                st_global_16(c_quadrant + (size_t)(i * 32 + row) * ldc + (lane % CH) * 8, v);
        }
    }
}

// Epilogue variants of the fp8 GEMM beyond "one scalar, bf16 out": per-row and per-column scales and the
// output element type.  The common case (no vectors, bf16) takes store_quadrant_bf16 above.
struct GemmEpilogue {
    float scale;                 // multiplies every element
    const float* row_scale;      // [M] or nullptr
    const float* col_scale;      // [N] or nullptr
    int out;                     // 0 = bf16, 1 = f32, 2 = e4m3 (round to nearest even, saturating at +-448)
    __device__ __host__ bool plain_bf16() const { return out == 0 && row_scale == nullptr && col_scale == nullptr; }
};
// One wave's 128x128 accumulator quadrant (layout as in store_quadrant_bf16) written straight from registers:
// a lane stores the 4 consecutive n of a register group of its row.  gm0 / gn0 = global row / column of the
// quadrant's first element; M, N = extents of C (row pitch N elements).
template <int NJ>
__device__ __forceinline__ void store_quadrant_ex(const f32x16 (&acc)[4][NJ], const GemmEpilogue& ep, void* C, int M, int N,
                                                  int gm0, int gn0, int lane) {
    const int r = lane & 31, g = lane >> 5;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = gm0 + i * 32 + r;
        if (gm >= M) continue;
        const float rs = ep.scale * (ep.row_scale ? ep.row_scale[gm] : 1.0f);
#pragma unroll
        for (int j = 0; j < NJ; ++j)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int gn = gn0 + j * 32 + q4 * 8 + g * 4;
                if (gn >= N) continue;                       // N is a multiple of 16: a group of 4 is inside or outside
                float v[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) v[x] = acc[i][j][q4 * 4 + x] * rs;
                if (ep.col_scale) {
                    const f32x4 cs = *reinterpret_cast<const f32x4*>(ep.col_scale + gn);
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] *= cs[x];
                }
                const size_t at = (size_t)gm * N + gn;
                if (ep.out == 1) {
                    *reinterpret_cast<f32x4*>(static_cast<float*>(C) + at) = f32x4{v[0], v[1], v[2], v[3]};
                } else if (ep.out == 2) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) v[x] = v[x] != v[x] ? v[x] : fminf(fmaxf(v[x], -448.0f), 448.0f);
                    int w = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
                    w = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], w, true);
                    *reinterpret_cast<int*>(static_cast<uint8_t*>(C) + at) = w;
                } else {
                    st_global_8(static_cast<uint16_t*>(C) + at, u32x2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])});
                }
            }
    }
}

// Grid remap for the 8 XCDs of an MI355X: consecutive workgroup ids are dealt round-robin
// to the XCDs, each with its own L2.  This returns a logical id such that the workgroups
// that land on one XCD cover one contiguous range of logical ids (so neighbours in the
// logical order share an L2).  Falls back to the identity when n is not a multiple of 8.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t pid, uint32_t n) {
    if (n % 8u) return pid;
    return (pid % 8u) * (n / 8u) + pid / 8u;
}

}  // namespace tyr
