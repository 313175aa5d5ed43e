// Internal launch entry points, one per kernel family.  All take validated arguments and
// return 0 on success, -1 if HIP reported a launch error.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace tyr {

// `batch` independent products; strides in elements between consecutive batch entries (stride_b = 0
// uses one B for every entry).
int launch_gemm_bf16(const void* a, const void* b, void* c, int M, int N, int K, int trans_b,
                     int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, hipStream_t stream);
// Process-wide switch that sends every GEMM shape through the general (register-staged) kernels.
// Its initial value is taken once from the environment variable TYR_HIP_GEMM_GENERAL.
bool gemm_general_only();
int set_gemm_general_only(int on);   // returns the previous value
// row_scale [M] / col_scale [N] (device f32, may be null); out_kind 0 = bf16, 1 = f32, 2 = e4m3
int launch_gemm_fp8(const void* aq, const void* bq, void* c, int M, int N, int K, float scale,
                    int trans_b, const float* row_scale, const float* col_scale, int out_kind, hipStream_t stream);
// Process-wide choice between persistent forward workgroups (two per CU walking the job ids) and one workgroup per job
// id.  Its initial value is taken once from the environment variable TYR_HIP_FA_PERSISTENT ("1" = persistent).
bool flash_attn_fwd_persistent();
int set_flash_attn_fwd_persistent(int on);   // returns the previous value
int launch_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                          int Hq, int Hkv, int N, int D, int causal, int window, const int* kv_lens,
                          const uint8_t* key_mask, float scale, hipStream_t stream);
size_t flash_attn_bwd_workspace_bytes(int B, int H, int N);
int launch_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                          const float* lse, void* dq, void* dk, void* dv, int B, int Hq, int Hkv, int N, int D,
                          int causal, int window, const int* kv_lens, const uint8_t* key_mask, float scale,
                          void* workspace, hipStream_t stream);
int launch_gqa_decode(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                      int Hq, int Hkv, int L, int D, int64_t kv_stride, float scale, int num_splits,
                      void* workspace, const int* kv_lens, int window, hipStream_t stream);

int launch_copy(const void* src, void* dst, size_t bytes, hipStream_t stream);
int launch_rope_fwd(const void* x, const float* cosp, const float* sinp, void* y, size_t rows, int S, int H, int D,
                    int is_bf16, hipStream_t stream);
int launch_decode_rope_append(const void* q, const void* k_new, const void* v_new, const float* cosp,
                              const float* sinp, void* q_out, void* k_cache, void* v_cache, int B, int Hq, int Hkv,
                              int D, size_t kv_stride, size_t pos, hipStream_t stream);
int launch_layernorm_residual(const void* x, const void* residual, const void* weight, const void* bias, void* out,
                              void* out_resid, size_t rows, int d_model, float eps, hipStream_t stream);

}  // namespace tyr
