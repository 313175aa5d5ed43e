// C ABI of the library (declared in include/tyr_hip.h): argument validation and dispatch.
// Validation mirrors what the reference's generated launchers check before a launch
// (Tyr/GPU/Codegen/Attribute.lean:331-386): every failure is reported through the return
// value, nothing throws, nothing is launched on invalid input.
#include "../../include/tyr_hip.h"

#include <hip/hip_runtime.h>
#include <limits.h>
#include <string.h>

#include <stdlib.h>

#include <atomic>
#include <mutex>

#include "launch.hpp"

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool fits_int(uint64_t v) { return v <= (uint64_t)INT_MAX; }

constexpr uint64_t kMaxSplits = 64;

uint64_t auto_splits(uint64_t B, uint64_t Hkv, uint64_t L) {
    // One workgroup (8 waves) per (batch, kv head) already fills the 256 CUs when there are at
    // least 256 such groups: then a single split is best (no partials, no second pass).  With
    // fewer groups the KV length is cut so that about 256 workgroups exist, as long as every wave
    // keeps at least two 32-row steps.
    const uint64_t groups = B * Hkv;
    if (groups == 0) return 1;
    uint64_t s = (256 + groups - 1) / groups;
    const uint64_t max_by_len = L / 512 ? L / 512 : 1;
    if (s > max_by_len) s = max_by_len;
    if (s < 1) s = 1;
    if (s > kMaxSplits) s = kMaxSplits;
    return s;
}

}  // namespace

// ---- process-wide switch between the fast and the general GEMM kernels (read on every GEMM launch,
// so it is an atomic flag; the environment is consulted once, when the flag is first needed)
namespace tyr {
static std::atomic<int> g_gemm_general{-1};          // -1 = not initialised
bool gemm_general_only() {
    int v = g_gemm_general.load(std::memory_order_relaxed);
    if (v < 0) {
        v = getenv("TYR_HIP_GEMM_GENERAL") != nullptr ? 1 : 0;
        int expected = -1;
        if (!g_gemm_general.compare_exchange_strong(expected, v)) v = expected;
    }
    return v != 0;
}
int set_gemm_general_only(int on) {
    const int prev = gemm_general_only() ? 1 : 0;
    g_gemm_general.store(on ? 1 : 0);
    return prev;
}
static std::atomic<int> g_fa_persistent{-1};         // -1 = not initialised
bool flash_attn_fwd_persistent() {
    int v = g_fa_persistent.load(std::memory_order_relaxed);
    if (v < 0) {
        const char* e = getenv("TYR_HIP_FA_PERSISTENT");
        v = (e != nullptr && e[0] == '1') ? 1 : 0;
        int expected = -1;
        if (!g_fa_persistent.compare_exchange_strong(expected, v)) v = expected;
    }
    return v != 0;
}
int set_flash_attn_fwd_persistent(int on) {
    const int prev = flash_attn_fwd_persistent() ? 1 : 0;
    g_fa_persistent.store(on ? 1 : 0);
    return prev;
}
}  // namespace tyr

// ---- the entry point that allocates nothing ---------------------------------------------------
// Partials of the split pass live in a file-scope device array.  Its name is only a host-side
// stand-in: the address a kernel may use is looked up once per device with hipGetSymbolAddress
// (every device holds its own copy of the array at its own address) and kept below.
constexpr size_t kStaticScratchBytes = TYR_HIP_GQA_DECODE_STATIC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices];            // device address of `scratch`, per device
static std::atomic<int> g_scratch_state[kMaxDevices];   // 0 = unresolved, 1 = resolved
static std::mutex g_scratch_mutex;

static int static_scratch(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return TYR_HIP_ERR_NO_DEVICE;
    }
    if (g_scratch_state[dev].load(std::memory_order_acquire) == 0) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_state[dev].load(std::memory_order_relaxed) == 0) {
            void* ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
                (void)hipGetLastError();
                return TYR_HIP_ERR_NO_DEVICE;
            }
            g_scratch_ptr[dev] = ptr;
            g_scratch_state[dev].store(1, std::memory_order_release);
        }
    }
    *out = g_scratch_ptr[dev];
    return TYR_HIP_OK;
}

extern "C" {

const char* tyr_hip_strerror(int status) {
    switch (status) {
        case TYR_HIP_OK: return "ok";
        case TYR_HIP_ERR_NULL_POINTER: return "a required tensor pointer is null";
        case TYR_HIP_ERR_BAD_SHAPE: return "tensor extents are zero, too large or inconsistent";
        case TYR_HIP_ERR_UNSUPPORTED: return "shape or option not supported by the gfx950 kernels";
        case TYR_HIP_ERR_MISALIGNED: return "tensor pointers and rows must be 16-byte aligned";
        case TYR_HIP_ERR_WORKSPACE: return "workspace is missing or too small";
        case TYR_HIP_ERR_LAUNCH: return "HIP reported a kernel launch error";
        case TYR_HIP_ERR_NO_DEVICE: return "no gfx950 device is available";
        case TYR_HIP_ERR_NOT_DEVICE_MEMORY: return "pointer must be a CUDA tensor (device memory)";
        default: return "unknown tyr_hip status";
    }
}

int tyr_hip_version(void) { return 100; }

int tyr_hip_device_info(int device, char* name, size_t name_len, int* compute_units,
                        int* lds_bytes_per_cu, int* clock_mhz, size_t* hbm_bytes) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) {
        (void)hipGetLastError();
        return TYR_HIP_ERR_NO_DEVICE;
    }
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, device) != hipSuccess) return TYR_HIP_ERR_NO_DEVICE;
    if (name && name_len) {
        strncpy(name, p.gcnArchName, name_len - 1);
        name[name_len - 1] = 0;
    }
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (lds_bytes_per_cu) *lds_bytes_per_cu = (int)p.maxSharedMemoryPerMultiProcessor;
    if (clock_mhz) *clock_mhz = p.clockRate / 1000;
    if (hbm_bytes) *hbm_bytes = p.totalGlobalMem;
    return TYR_HIP_OK;
}

int tyr_hip_check_device_pointer(const void* p) {
    if (!p) return TYR_HIP_ERR_NULL_POINTER;
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return TYR_HIP_ERR_NOT_DEVICE_MEMORY;
    }
    return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged
               ? TYR_HIP_OK
               : TYR_HIP_ERR_NOT_DEVICE_MEMORY;
}

int tyr_hip_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                           uint64_t B, uint64_t H, uint64_t N, uint64_t D, int causal, float scale,
                           void* stream) {
    return tyr_hip_flash_attn_fwd_gqa(q, k, v, o, lse, B, H, H, N, D, causal, 0, nullptr, scale, stream);
}

static int attn_fwd_checked(const void* q, const void* k, const void* v, void* o, float* lse,
                            uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                            int causal, uint64_t window, const int32_t* kv_lens, const uint8_t* key_mask,
                            float scale, void* stream) {
    if (!q || !k || !v || !o) return TYR_HIP_ERR_NULL_POINTER;
    if (B == 0 || Hq == 0 || Hkv == 0 || N == 0 || D == 0 || Hq % Hkv != 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return TYR_HIP_ERR_UNSUPPORTED;
    if (window > 0 && !causal) return TYR_HIP_ERR_UNSUPPORTED;        // the window is a causal one
    if (!(scale > 0.0f) || scale > 3.0e38f) return TYR_HIP_ERR_UNSUPPORTED;
    if (!fits_int(N) || !fits_int(B * Hq) || B * Hq > (uint64_t)INT_MAX / ((N + 127) / 128))
        return TYR_HIP_ERR_BAD_SHAPE;
    if (N * D * 2 >= ((uint64_t)1 << 32)) return TYR_HIP_ERR_UNSUPPORTED;   // one head's K or V must stay below 4 GiB
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return TYR_HIP_ERR_MISALIGNED;
    if (lse && (reinterpret_cast<uintptr_t>(lse) & 3u)) return TYR_HIP_ERR_MISALIGNED;
    if (kv_lens && (reinterpret_cast<uintptr_t>(kv_lens) & 3u)) return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_flash_attn_fwd(q, k, v, o, lse, (int)B, (int)Hq, (int)Hkv, (int)N, (int)D,
                                              causal != 0, (int)(window > (uint64_t)INT_MAX ? INT_MAX : window),
                                              kv_lens, key_mask, scale, static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_flash_attn_fwd_gqa(const void* q, const void* k, const void* v, void* o, float* lse,
                               uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                               int causal, uint64_t window, const int32_t* kv_lens, float scale,
                               void* stream) {
    return attn_fwd_checked(q, k, v, o, lse, B, Hq, Hkv, N, D, causal, window, kv_lens, nullptr, scale, stream);
}

int tyr_hip_flash_attn_fwd_mask(const void* q, const void* k, const void* v, void* o, float* lse,
                                uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                int causal, const uint8_t* key_mask, float scale, void* stream) {
    if (!key_mask) return TYR_HIP_ERR_NULL_POINTER;
    return attn_fwd_checked(q, k, v, o, lse, B, Hq, Hkv, N, D, causal, 0, nullptr, key_mask, scale, stream);
}

size_t tyr_hip_flash_attn_bwd_workspace_bytes(uint64_t B, uint64_t H, uint64_t N, uint64_t D) {
    (void)D;
    if (!fits_int(N) || !fits_int(B * H)) return 0;
    return tyr::flash_attn_bwd_workspace_bytes((int)B, (int)H, (int)N);
}

int tyr_hip_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o,
                           const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                           uint64_t B, uint64_t H, uint64_t N, uint64_t D, int causal, float scale,
                           void* workspace, size_t workspace_bytes, void* stream) {
    return tyr_hip_flash_attn_bwd_gqa(q, k, v, o, d_o, lse, dq, dk, dv, B, H, H, N, D, causal, 0, nullptr, scale,
                                      workspace, workspace_bytes, stream);
}

static int attn_bwd_checked(const void* q, const void* k, const void* v, const void* o,
                            const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                            uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                            int causal, uint64_t window, const int32_t* kv_lens, const uint8_t* key_mask,
                            float scale, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !o || !d_o || !lse || !dq || !dk || !dv) return TYR_HIP_ERR_NULL_POINTER;
    if (B == 0 || Hq == 0 || Hkv == 0 || N == 0 || D == 0 || Hq % Hkv != 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (D != 64 && D != 128) return TYR_HIP_ERR_UNSUPPORTED;
    if (window > 0 && !causal) return TYR_HIP_ERR_UNSUPPORTED;
    if (!(scale > 0.0f) || scale > 3.0e38f) return TYR_HIP_ERR_UNSUPPORTED;
    if (!fits_int(N) || !fits_int(B * Hq) || B * Hq > (uint64_t)INT_MAX / ((N + 127) / 128))
        return TYR_HIP_ERR_BAD_SHAPE;
    // 32-bit offsets inside the G query heads of one kv head (and inside their pairs)
    if ((Hq / Hkv) * N * D * 2 >= ((uint64_t)1 << 31)) return TYR_HIP_ERR_UNSUPPORTED;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(d_o) ||
        !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
        return TYR_HIP_ERR_MISALIGNED;
    if (reinterpret_cast<uintptr_t>(lse) & 3u) return TYR_HIP_ERR_MISALIGNED;
    if (kv_lens && (reinterpret_cast<uintptr_t>(kv_lens) & 3u)) return TYR_HIP_ERR_MISALIGNED;
    const size_t need = tyr_hip_flash_attn_bwd_workspace_bytes(B, Hq, N, D);
    if (!workspace || workspace_bytes < need) return TYR_HIP_ERR_WORKSPACE;
    if (!aligned16(workspace)) return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_flash_attn_bwd(q, k, v, o, d_o, lse, dq, dk, dv, (int)B, (int)Hq, (int)Hkv, (int)N,
                                              (int)D, causal != 0,
                                              (int)(window > (uint64_t)INT_MAX ? INT_MAX : window), kv_lens, key_mask,
                                              scale, workspace, static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_flash_attn_bwd_gqa(const void* q, const void* k, const void* v, const void* o,
                               const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                               uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                               int causal, uint64_t window, const int32_t* kv_lens, float scale,
                               void* workspace, size_t workspace_bytes, void* stream) {
    return attn_bwd_checked(q, k, v, o, d_o, lse, dq, dk, dv, B, Hq, Hkv, N, D, causal, window, kv_lens, nullptr,
                            scale, workspace, workspace_bytes, stream);
}

int tyr_hip_flash_attn_bwd_mask(const void* q, const void* k, const void* v, const void* o,
                                const void* d_o, const float* lse, void* dq, void* dk, void* dv,
                                uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                int causal, const uint8_t* key_mask, float scale,
                                void* workspace, size_t workspace_bytes, void* stream) {
    if (!key_mask) return TYR_HIP_ERR_NULL_POINTER;
    return attn_bwd_checked(q, k, v, o, d_o, lse, dq, dk, dv, B, Hq, Hkv, N, D, causal, 0, nullptr, key_mask,
                            scale, workspace, workspace_bytes, stream);
}

uint64_t tyr_hip_gqa_decode_auto_splits(uint64_t B, uint64_t Hkv, uint64_t L) {
    return auto_splits(B, Hkv, L);
}

size_t tyr_hip_gqa_decode_workspace_bytes(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L,
                                          uint64_t D, uint64_t num_splits) {
    if (num_splits == 0) num_splits = auto_splits(B, Hkv, L);
    return (size_t)(B * Hq * num_splits * (D + 2) * sizeof(float));
}

int tyr_hip_gqa_decode(const void* q, const void* k, const void* v, void* o, float* lse,
                       uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                       uint64_t kv_stride, float scale, uint64_t num_splits, void* workspace,
                       size_t workspace_bytes, void* stream) {
    return tyr_hip_gqa_decode_varlen(q, k, v, o, lse, B, Hq, Hkv, L, D, kv_stride, nullptr, 0, scale,
                                     num_splits, workspace, workspace_bytes, stream);
}

int tyr_hip_gqa_decode_varlen(const void* q, const void* k, const void* v, void* o, float* lse,
                              uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                              uint64_t kv_stride, const int32_t* kv_lens, uint64_t window, float scale,
                              uint64_t num_splits, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !o) return TYR_HIP_ERR_NULL_POINTER;
    if (B == 0 || Hq == 0 || Hkv == 0 || L == 0 || D == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (Hq % Hkv != 0 || kv_stride < L) return TYR_HIP_ERR_BAD_SHAPE;
    if ((D != 128 && D != 64) || Hq / Hkv > 16 || num_splits > kMaxSplits) return TYR_HIP_ERR_UNSUPPORTED;
    if (!(scale > 0.0f) || scale > 3.0e38f) return TYR_HIP_ERR_UNSUPPORTED;
    if (!fits_int(L) || !fits_int(B * Hq) || kv_stride > (uint64_t)INT_MAX) return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o)) return TYR_HIP_ERR_MISALIGNED;
    if (kv_lens && (reinterpret_cast<uintptr_t>(kv_lens) & 3u)) return TYR_HIP_ERR_MISALIGNED;
    if (num_splits == 0) num_splits = auto_splits(B, Hkv, window > 0 && window < L ? window : L);
    if (!fits_int(B * Hkv * num_splits)) return TYR_HIP_ERR_BAD_SHAPE;      // one workgroup per (group, split)
    const size_t need = tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, L, D, num_splits);
    if (!workspace || workspace_bytes < need) return TYR_HIP_ERR_WORKSPACE;
    if (!aligned16(workspace)) return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_gqa_decode(q, k, v, o, lse, (int)B, (int)Hq, (int)Hkv, (int)L, (int)D,
                                          (int64_t)kv_stride, scale, (int)num_splits, workspace, kv_lens,
                                          (int)(window > (uint64_t)INT_MAX ? INT_MAX : window),
                                          static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_gqa_decode_static(const void* q, const void* k, const void* v, void* o, float* lse,
                              uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                              uint64_t kv_stride, float scale, uint64_t num_splits, void* stream) {
    // sizes are judged before anything touches the device, so an oversized request is an error
    // return and never a launch
    if (B == 0 || Hq == 0 || Hkv == 0 || L == 0 || D == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (num_splits > kMaxSplits) return TYR_HIP_ERR_UNSUPPORTED;
    if (B > (uint64_t)INT_MAX || Hq > (uint64_t)INT_MAX || B * Hq > (uint64_t)INT_MAX || Hkv > Hq || D > 4096)
        return TYR_HIP_ERR_BAD_SHAPE;
    const size_t need = tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, L, D, num_splits);
    if (need > kStaticScratchBytes) return TYR_HIP_ERR_WORKSPACE;
    void* ptr = nullptr;
    const int rc = static_scratch(&ptr);
    if (rc != TYR_HIP_OK) return rc;
    return tyr_hip_gqa_decode_varlen(q, k, v, o, lse, B, Hq, Hkv, L, D, kv_stride, nullptr, 0, scale, num_splits,
                                     ptr, kStaticScratchBytes, stream);
}

int tyr_hip_decode_rope_append(const void* q, const void* k_new, const void* v_new, const float* cos,
                               const float* sin, void* q_out, void* k_cache, void* v_cache, uint64_t B,
                               uint64_t Hq, uint64_t Hkv, uint64_t D, uint64_t kv_stride, uint64_t pos,
                               void* stream) {
    if (!q || !k_new || !v_new || !cos || !sin || !q_out || !k_cache || !v_cache) return TYR_HIP_ERR_NULL_POINTER;
    if (B == 0 || Hq == 0 || Hkv == 0 || D == 0 || pos >= kv_stride) return TYR_HIP_ERR_BAD_SHAPE;
    if (D % 16 != 0) return TYR_HIP_ERR_UNSUPPORTED;
    if (!fits_int(D) || !fits_int(B * Hq) || !fits_int(B * Hkv) || !fits_int((B * Hq + 2 * B * Hkv) * (D / 16)))
        return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(q) || !aligned16(k_new) || !aligned16(v_new) || !aligned16(cos) || !aligned16(sin) ||
        !aligned16(q_out) || !aligned16(k_cache) || !aligned16(v_cache))
        return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_decode_rope_append(q, k_new, v_new, cos, sin, q_out, k_cache, v_cache, (int)B,
                                                  (int)Hq, (int)Hkv, (int)D, (size_t)kv_stride, (size_t)pos,
                                                  static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_rope_fwd(const void* x, const float* cos, const float* sin, void* y, uint64_t B, uint64_t S,
                     uint64_t H, uint64_t D, int dtype, void* stream) {
    if (!x || !cos || !sin || !y) return TYR_HIP_ERR_NULL_POINTER;
    if (B == 0 || S == 0 || H == 0 || D == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (dtype != TYR_HIP_F32 && dtype != TYR_HIP_BF16) return TYR_HIP_ERR_UNSUPPORTED;
    if (D % (dtype == TYR_HIP_BF16 ? 16 : 8) != 0) return TYR_HIP_ERR_UNSUPPORTED;
    if (!fits_int(S) || !fits_int(H) || !fits_int(D)) return TYR_HIP_ERR_BAD_SHAPE;
    const uint64_t rows = B * S * H;
    if (rows / S / H != B || rows * (D / 8) / rows != D / 8 || rows * (D / 8) / 256 > (uint64_t)INT_MAX)
        return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(cos) || !aligned16(sin) || !aligned16(y)) return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_rope_fwd(x, cos, sin, y, (size_t)rows, (int)S, (int)H, (int)D,
                                        dtype == TYR_HIP_BF16, static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_layernorm_residual(const void* x, const void* residual, const void* weight, const void* bias,
                               void* out, void* out_resid, uint64_t rows, uint64_t d_model, float eps,
                               void* stream) {
    if (!x || !residual || !weight || !bias || !out || !out_resid) return TYR_HIP_ERR_NULL_POINTER;
    if (rows == 0 || d_model == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (d_model % 8 != 0 || d_model > 8192 || !(eps >= 0.0f)) return TYR_HIP_ERR_UNSUPPORTED;
    if ((rows + 3) / 4 > (uint64_t)INT_MAX) return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(residual) || !aligned16(weight) || !aligned16(bias) || !aligned16(out) ||
        !aligned16(out_resid))
        return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_layernorm_residual(x, residual, weight, bias, out, out_resid, (size_t)rows,
                                                  (int)d_model, eps, static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_copy(const void* src, void* dst, size_t bytes, void* stream) {
    if (!src || !dst) return TYR_HIP_ERR_NULL_POINTER;
    if (bytes == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (!aligned16(src) || !aligned16(dst)) return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_copy(src, dst, bytes, static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_gemm_bf16(const void* a, const void* b, void* c, uint64_t M, uint64_t N, uint64_t K,
                      int trans_b, void* stream) {
    return tyr_hip_gemm_bf16_batched(a, b, c, 1, M, N, K, 0, 0, 0, trans_b, stream);
}

int tyr_hip_gemm_bf16_batched(const void* a, const void* b, void* c, uint64_t batch, uint64_t M, uint64_t N,
                              uint64_t K, uint64_t stride_a, uint64_t stride_b, uint64_t stride_c, int trans_b,
                              void* stream) {
    if (!a || !b || !c) return TYR_HIP_ERR_NULL_POINTER;
    if (batch == 0 || M == 0 || N == 0 || K == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (!fits_int(M) || !fits_int(N) || !fits_int(K) || batch > 65535) return TYR_HIP_ERR_BAD_SHAPE;
    if (((M + 255) / 256) * ((N + 255) / 256) > (uint64_t)INT_MAX) return TYR_HIP_ERR_BAD_SHAPE;
    if (K % 8 != 0 || N % 8 != 0) return TYR_HIP_ERR_UNSUPPORTED;
    if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return TYR_HIP_ERR_MISALIGNED;
    if (batch > 1) {
        // every batch entry keeps 16-byte alignment; outputs of different entries must not overlap
        if (stride_a % 8 != 0 || stride_b % 8 != 0 || stride_c % 8 != 0) return TYR_HIP_ERR_MISALIGNED;
        if (stride_c < M * N) return TYR_HIP_ERR_BAD_SHAPE;
        if (stride_a > ((uint64_t)1 << 40) || stride_b > ((uint64_t)1 << 40) || stride_c > ((uint64_t)1 << 40))
            return TYR_HIP_ERR_BAD_SHAPE;
    }
    const int rc = tyr::launch_gemm_bf16(a, b, c, (int)M, (int)N, (int)K, trans_b != 0, (int)batch,
                                         (int64_t)stride_a, (int64_t)stride_b, (int64_t)stride_c,
                                         static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

int tyr_hip_gemm_force_general(int on) { return tyr::set_gemm_general_only(on); }

int tyr_hip_flash_attn_fwd_persistent(int on) { return tyr::set_flash_attn_fwd_persistent(on); }

int tyr_hip_gemm_fp8(const void* aq, const void* bq, void* c, uint64_t M, uint64_t N, uint64_t K,
                     float scale_a, float scale_b, int trans_b, void* stream) {
    return tyr_hip_gemm_fp8_ex(aq, bq, c, M, N, K, scale_a * scale_b, nullptr, nullptr, TYR_HIP_OUT_BF16, trans_b, stream);
}

int tyr_hip_gemm_fp8_ex(const void* aq, const void* bq, void* c, uint64_t M, uint64_t N, uint64_t K,
                        float scale, const float* row_scale, const float* col_scale, int out_dtype,
                        int trans_b, void* stream) {
    if (!aq || !bq || !c) return TYR_HIP_ERR_NULL_POINTER;
    if (M == 0 || N == 0 || K == 0) return TYR_HIP_ERR_BAD_SHAPE;
    if (!fits_int(M) || !fits_int(N) || !fits_int(K)) return TYR_HIP_ERR_BAD_SHAPE;
    if (((M + 255) / 256) * ((N + 255) / 256) > (uint64_t)INT_MAX) return TYR_HIP_ERR_BAD_SHAPE;
    if (K % 16 != 0 || N % 16 != 0) return TYR_HIP_ERR_UNSUPPORTED;
    if (out_dtype != TYR_HIP_OUT_BF16 && out_dtype != TYR_HIP_OUT_F32 && out_dtype != TYR_HIP_OUT_E4M3)
        return TYR_HIP_ERR_UNSUPPORTED;
    if (!aligned16(aq) || !aligned16(bq) || !aligned16(c)) return TYR_HIP_ERR_MISALIGNED;
    if ((row_scale && (reinterpret_cast<uintptr_t>(row_scale) & 3u)) || (col_scale && !aligned16(col_scale)))
        return TYR_HIP_ERR_MISALIGNED;
    const int rc = tyr::launch_gemm_fp8(aq, bq, c, (int)M, (int)N, (int)K, scale, trans_b != 0, row_scale, col_scale,
                                        out_dtype, static_cast<hipStream_t>(stream));
    return rc == 0 ? TYR_HIP_OK : TYR_HIP_ERR_LAUNCH;
}

}  // extern "C"
