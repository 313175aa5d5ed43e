// Internal launch entry points, one per kernel family.  All take validated arguments and
// return 0 on success, -1 if HIP reported a launch error.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace tyr {

int launch_gemm_bf16(const void* a, const void* b, void* c, int M, int N, int K, int trans_b,
                     hipStream_t stream);
int launch_gemm_fp8(const void* aq, const void* bq, void* c, int M, int N, int K, float scale,
                    int trans_b, hipStream_t stream);
int launch_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                          int H, int N, int D, int causal, float scale, hipStream_t stream);
size_t flash_attn_bwd_workspace_bytes(int B, int H, int N);
int launch_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o,
                          const float* lse, void* dq, void* dk, void* dv, int B, int H, int N, int D,
                          int causal, float scale, void* workspace, hipStream_t stream);
int launch_gqa_decode(const void* q, const void* k, const void* v, void* o, float* lse, int B,
                      int Hq, int Hkv, int L, int D, int64_t kv_stride, float scale, int num_splits,
                      void* workspace, hipStream_t stream);

}  // namespace tyr
