// Lean-facing wrappers over the C ABI in include/tyr_hip.h.
//
// These are the symbols the `@[extern]` declarations in lean/Tyr/GPU/GFX950.lean bind.  They
// follow the conventions of the reference's FFI:
//   * tensor arguments are *borrowed* Lean external objects wrapping a c10::TensorImpl
//     (`borrowTensor`, cc/src/tyr.cpp:127-148); results are handed to Lean with `giveTensor`
//     (cc/src/tyr.cpp:152-160);
//   * implicit `{B H N D : UInt64}` binders arrive first as unboxed uint64_t
//     (cc/src/tyr.cpp:3913-3918), Lean `Float` is C double, `Bool` is uint8_t
//     (cc/src/tyr.cpp:2571-2572);
//   * errors never cross the boundary as C++ exceptions: they become
//     `IO.userError msg` (Tyr/GPU/Codegen/Attribute.lean:373-386), with the launcher's own
//     messages "<p> must be a CUDA tensor" / "<p> must be contiguous" / "<p> must have dim <= 4"
//     (Tyr/GPU/Codegen/Attribute.lean:334-336);
//   * a pair is returned as `lean_alloc_ctor(0, 2, 0)` (cc/src/tyr.cpp:4275-4283) inside
//     `lean_io_result_mk_ok`; the trailing IO world token is declared explicitly.
//
// The file is compiled into libTyrC only where <lean/lean.h> and LibTorch headers exist (the
// reference's `make -C cc`); nothing else in this library depends on Lean or torch.
#if defined(__has_include)
#if __has_include(<lean/lean.h>) && __has_include(<torch/torch.h>)
#define TYR_HAVE_LEAN 1
#endif
#endif

#ifdef TYR_HAVE_LEAN
#include <lean/lean.h>
#include <torch/torch.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <cmath>
#include <string>

#include "../../include/tyr_hip.h"

// Provided by the reference's cc/src/tyr.cpp (same library).
torch::Tensor borrowTensor(b_lean_obj_arg o);
lean_object* giveTensor(torch::Tensor t);

namespace {

lean_object* io_error(const std::string& msg) {
    return lean_io_result_mk_error(lean_mk_io_user_error(lean_mk_string(msg.c_str())));
}

// The reference launcher's three checks, plus the dtype the kernel expects.
bool check(const torch::Tensor& t, const char* name, c10::ScalarType dt, std::string& err) {
    if (!t.is_cuda()) { err = std::string(name) + " must be a CUDA tensor"; return false; }
    if (!t.is_contiguous()) { err = std::string(name) + " must be contiguous"; return false; }
    if (t.dim() > 4) { err = std::string(name) + " must have dim <= 4"; return false; }
    if (t.scalar_type() != dt) { err = std::string(name) + " has the wrong dtype"; return false; }
    return true;
}

// Outputs and scratch are allocated by LibTorch's caching allocator, which hands a freed block to
// the next allocation on the stream it was allocated on.  The kernels run on the caller's `stream`,
// so for the duration of a call that stream is made LibTorch's current one: the blocks then belong
// to it, and a scratch tensor dropped at the end of the call (while its kernels are still queued)
// can only be reused by work queued behind them on the same stream.
struct LaunchStreamScope {
    static c10::hip::HIPStreamMasqueradingAsCUDA wrap(uint64_t stream, c10::DeviceIndex dev) {
        return stream ? c10::hip::getStreamFromExternalMasqueradingAsCUDA(reinterpret_cast<hipStream_t>(stream), dev)
                      : c10::hip::getDefaultHIPStreamMasqueradingAsCUDA(dev);
    }
    c10::hip::HIPStreamGuardMasqueradingAsCUDA guard;
    LaunchStreamScope(uint64_t stream, const torch::Tensor& like) : guard(wrap(stream, like.device().index())) {}
};

lean_object* pair_result(torch::Tensor a, torch::Tensor b) {
    lean_object* p = lean_alloc_ctor(0, 2, 0);
    lean_ctor_set(p, 0, giveTensor(std::move(a)));
    lean_ctor_set(p, 1, giveTensor(std::move(b)));
    return lean_io_result_mk_ok(p);
}

lean_object* status_error(const char* what, int rc) {
    return io_error(std::string(what) + ": " + tyr_hip_strerror(rc));
}

}  // namespace

extern "C" {

// flashAttnFwd {B H N D} q k v causal scale stream : IO (T #[B,H,N,D] x T #[B,H,N])
lean_object* lean_tyr_gpu_flash_attn_fwd(uint64_t B, uint64_t H, uint64_t N, uint64_t D,
                                         b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                         uint8_t causal, double scale, uint64_t stream,
                                         lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto o = torch::empty_like(q_);
        auto lse = torch::empty({(int64_t)B, (int64_t)H, (int64_t)N}, q_.options().dtype(torch::kFloat32));
        const int rc = tyr_hip_flash_attn_fwd(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr(),
                                              lse.data_ptr<float>(), B, H, N, D, causal, (float)scale,
                                              reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnFwd", rc);
        return pair_result(std::move(o), std::move(lse));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnFwdGQA {B Hq Hkv N D} q k v kvLens causal window scale stream : IO (T #[B,Hq,N,D] x T #[B,Hq,N])
lean_object* lean_tyr_gpu_flash_attn_fwd_gqa(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                             b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                             b_lean_obj_arg kv_lens, uint8_t causal, uint64_t window, double scale,
                                             uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), n_ = borrowTensor(kv_lens);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(n_, "kvLens", torch::kInt32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto o = torch::empty_like(q_);
        auto lse = torch::empty({(int64_t)B, (int64_t)Hq, (int64_t)N}, q_.options().dtype(torch::kFloat32));
        const int rc = tyr_hip_flash_attn_fwd_gqa(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr(),
                                                  lse.data_ptr<float>(), B, Hq, Hkv, N, D, causal, window,
                                                  n_.data_ptr<int32_t>(), (float)scale, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnFwdGQA", rc);
        return pair_result(std::move(o), std::move(lse));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnFwdGQAFull: flashAttnFwdGQA for sequences that all have N keys (no length tensor, so the launch takes the
// kernel without the length and window instructions when window = 0).
// flashAttnFwdGQAFull {B Hq Hkv N D} q k v causal window scale stream : IO (T #[B,Hq,N,D] x T #[B,Hq,N])
lean_object* lean_tyr_gpu_flash_attn_fwd_gqa_full(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                             b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                             uint8_t causal, uint64_t window, double scale,
                                             uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto o = torch::empty_like(q_);
        auto lse = torch::empty({(int64_t)B, (int64_t)Hq, (int64_t)N}, q_.options().dtype(torch::kFloat32));
        const int rc = tyr_hip_flash_attn_fwd_gqa(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr(),
                                                  lse.data_ptr<float>(), B, Hq, Hkv, N, D, causal, window,
                                                  nullptr, (float)scale, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnFwdGQA", rc);
        return pair_result(std::move(o), std::move(lse));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnBwd {B H N D} q k v o lse dO causal scale stream : IO (dQ x dK x dV)
// The triple is returned as the nested pair (dQ, (dK, dV)), Lean's representation of a x b x c.
lean_object* lean_tyr_gpu_flash_attn_bwd(uint64_t B, uint64_t H, uint64_t N, uint64_t D,
                                         b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                         b_lean_obj_arg o, b_lean_obj_arg lse, b_lean_obj_arg d_o,
                                         uint8_t causal, double scale, uint64_t stream,
                                         lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), o_ = borrowTensor(o);
        auto lse_ = borrowTensor(lse), g_ = borrowTensor(d_o);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(o_, "o", torch::kBFloat16, err) ||
            !check(g_, "dO", torch::kBFloat16, err) || !check(lse_, "lse", torch::kFloat32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto dq = torch::empty_like(q_), dk = torch::empty_like(q_), dv = torch::empty_like(q_);
        const size_t ws_bytes = tyr_hip_flash_attn_bwd_workspace_bytes(B, H, N, D);
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, q_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_flash_attn_bwd(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o_.data_ptr(),
                                              g_.data_ptr(), lse_.data_ptr<float>(), dq.data_ptr(),
                                              dk.data_ptr(), dv.data_ptr(), B, H, N, D, causal, (float)scale,
                                              ws.data_ptr(), ws_bytes, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnBwd", rc);
        lean_object* inner = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(inner, 0, giveTensor(std::move(dk)));
        lean_ctor_set(inner, 1, giveTensor(std::move(dv)));
        lean_object* outer = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(outer, 0, giveTensor(std::move(dq)));
        lean_ctor_set(outer, 1, inner);
        return lean_io_result_mk_ok(outer);
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnBwdGQA {B Hq Hkv N D} q k v o lse dO kvLens causal window scale stream : IO (dQ x dK x dV)
lean_object* lean_tyr_gpu_flash_attn_bwd_gqa(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                             b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                             b_lean_obj_arg o, b_lean_obj_arg lse, b_lean_obj_arg d_o,
                                             b_lean_obj_arg kv_lens, uint8_t causal, uint64_t window, double scale,
                                             uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), o_ = borrowTensor(o);
        auto lse_ = borrowTensor(lse), g_ = borrowTensor(d_o), n_ = borrowTensor(kv_lens);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(o_, "o", torch::kBFloat16, err) ||
            !check(g_, "dO", torch::kBFloat16, err) || !check(lse_, "lse", torch::kFloat32, err) ||
            !check(n_, "kvLens", torch::kInt32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto dq = torch::empty_like(q_), dk = torch::empty_like(k_), dv = torch::empty_like(k_);
        const size_t ws_bytes = tyr_hip_flash_attn_bwd_workspace_bytes(B, Hq, N, D);
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, q_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_flash_attn_bwd_gqa(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o_.data_ptr(),
                                                  g_.data_ptr(), lse_.data_ptr<float>(), dq.data_ptr(), dk.data_ptr(),
                                                  dv.data_ptr(), B, Hq, Hkv, N, D, causal, window,
                                                  n_.data_ptr<int32_t>(), (float)scale, ws.data_ptr(), ws_bytes,
                                                  reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnBwdGQA", rc);
        lean_object* inner = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(inner, 0, giveTensor(std::move(dk)));
        lean_ctor_set(inner, 1, giveTensor(std::move(dv)));
        lean_object* outer = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(outer, 0, giveTensor(std::move(dq)));
        lean_ctor_set(outer, 1, inner);
        return lean_io_result_mk_ok(outer);
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnBwdGQAFull {B Hq Hkv N D} q k v o lse dO causal window scale stream : IO (dQ x dK x dV)
lean_object* lean_tyr_gpu_flash_attn_bwd_gqa_full(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                             b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                             b_lean_obj_arg o, b_lean_obj_arg lse, b_lean_obj_arg d_o,
                                             uint8_t causal, uint64_t window, double scale,
                                             uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), o_ = borrowTensor(o);
        auto lse_ = borrowTensor(lse), g_ = borrowTensor(d_o);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(o_, "o", torch::kBFloat16, err) ||
            !check(g_, "dO", torch::kBFloat16, err) || !check(lse_, "lse", torch::kFloat32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto dq = torch::empty_like(q_), dk = torch::empty_like(k_), dv = torch::empty_like(k_);
        const size_t ws_bytes = tyr_hip_flash_attn_bwd_workspace_bytes(B, Hq, N, D);
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, q_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_flash_attn_bwd_gqa(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o_.data_ptr(),
                                                  g_.data_ptr(), lse_.data_ptr<float>(), dq.data_ptr(), dk.data_ptr(),
                                                  dv.data_ptr(), B, Hq, Hkv, N, D, causal, window,
                                                  nullptr, (float)scale, ws.data_ptr(), ws_bytes,
                                                  reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnBwdGQA", rc);
        lean_object* inner = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(inner, 0, giveTensor(std::move(dk)));
        lean_ctor_set(inner, 1, giveTensor(std::move(dv)));
        lean_object* outer = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(outer, 0, giveTensor(std::move(dq)));
        lean_ctor_set(outer, 1, inner);
        return lean_io_result_mk_ok(outer);
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnFwdMask {B Hq Hkv N D} q k v keyMask causal scale stream : IO (T #[B,Hq,N,D] x T #[B,Hq,N])
// keyMask : uint8 [B, N], nonzero = visible key (the mask argument of lean_torch_sdpa_gqa_mask as bytes)
lean_object* lean_tyr_gpu_flash_attn_fwd_mask(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                              b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                              b_lean_obj_arg key_mask, uint8_t causal, double scale,
                                              uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), m_ = borrowTensor(key_mask);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(m_, "keyMask", torch::kUInt8, err))
            return io_error(err);
        if ((uint64_t)m_.numel() != B * N) return io_error("flashAttnFwdMask: keyMask must hold B*N bytes");
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto o = torch::empty_like(q_);
        auto lse = torch::empty({(int64_t)B, (int64_t)Hq, (int64_t)N}, q_.options().dtype(torch::kFloat32));
        const int rc = tyr_hip_flash_attn_fwd_mask(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr(),
                                                   lse.data_ptr<float>(), B, Hq, Hkv, N, D, causal,
                                                   m_.data_ptr<uint8_t>(), (float)scale,
                                                   reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnFwdMask", rc);
        return pair_result(std::move(o), std::move(lse));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// flashAttnBwdMask {B Hq Hkv N D} q k v o lse dO keyMask causal scale stream : IO (dQ x dK x dV)
lean_object* lean_tyr_gpu_flash_attn_bwd_mask(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t N, uint64_t D,
                                              b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                              b_lean_obj_arg o, b_lean_obj_arg lse, b_lean_obj_arg d_o,
                                              b_lean_obj_arg key_mask, uint8_t causal, double scale,
                                              uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), o_ = borrowTensor(o);
        auto lse_ = borrowTensor(lse), g_ = borrowTensor(d_o), m_ = borrowTensor(key_mask);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(o_, "o", torch::kBFloat16, err) ||
            !check(g_, "dO", torch::kBFloat16, err) || !check(lse_, "lse", torch::kFloat32, err) ||
            !check(m_, "keyMask", torch::kUInt8, err))
            return io_error(err);
        if ((uint64_t)m_.numel() != B * N) return io_error("flashAttnBwdMask: keyMask must hold B*N bytes");
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto dq = torch::empty_like(q_), dk = torch::empty_like(k_), dv = torch::empty_like(k_);
        const size_t ws_bytes = tyr_hip_flash_attn_bwd_workspace_bytes(B, Hq, N, D);
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, q_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_flash_attn_bwd_mask(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o_.data_ptr(),
                                                   g_.data_ptr(), lse_.data_ptr<float>(), dq.data_ptr(),
                                                   dk.data_ptr(), dv.data_ptr(), B, Hq, Hkv, N, D, causal,
                                                   m_.data_ptr<uint8_t>(), (float)scale, ws.data_ptr(), ws_bytes,
                                                   reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("flashAttnBwdMask", rc);
        lean_object* inner = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(inner, 0, giveTensor(std::move(dk)));
        lean_ctor_set(inner, 1, giveTensor(std::move(dv)));
        lean_object* outer = lean_alloc_ctor(0, 2, 0);
        lean_ctor_set(outer, 0, giveTensor(std::move(dq)));
        lean_ctor_set(outer, 1, inner);
        return lean_io_result_mk_ok(outer);
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gqaDecode {B Hq Hkv L D} q k v scale numSplits stream : IO (T #[B,Hq,1,D] x T #[B,Hq])
lean_object* lean_tyr_gpu_gqa_decode(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                                     b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v, double scale,
                                     uint64_t num_splits, uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto o = torch::empty_like(q_);
        auto lse = torch::empty({(int64_t)B, (int64_t)Hq}, q_.options().dtype(torch::kFloat32));
        const size_t ws_bytes = tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, L, D, num_splits);
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, q_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_gqa_decode(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr(),
                                          lse.data_ptr<float>(), B, Hq, Hkv, L, D, /*kv_stride=*/L,
                                          (float)scale, num_splits, ws.data_ptr(), ws_bytes,
                                          reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gqaDecode", rc);
        return pair_result(std::move(o), std::move(lse));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gqaDecodeVarlen {B Hq Hkv L D} q k v kvLens window scale numSplits stream : IO (T #[B,Hq,1,D] x T #[B,Hq])
lean_object* lean_tyr_gpu_gqa_decode_varlen(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                                            b_lean_obj_arg q, b_lean_obj_arg k, b_lean_obj_arg v,
                                            b_lean_obj_arg kv_lens, uint64_t window, double scale,
                                            uint64_t num_splits, uint64_t stream, lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), k_ = borrowTensor(k), v_ = borrowTensor(v), n_ = borrowTensor(kv_lens);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(k_, "k", torch::kBFloat16, err) ||
            !check(v_, "v", torch::kBFloat16, err) || !check(n_, "kvLens", torch::kInt32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto o = torch::empty_like(q_);
        auto lse = torch::empty({(int64_t)B, (int64_t)Hq}, q_.options().dtype(torch::kFloat32));
        const size_t ws_bytes = tyr_hip_gqa_decode_workspace_bytes(B, Hq, Hkv, L, D, num_splits);
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, q_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_gqa_decode_varlen(q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), o.data_ptr(),
                                                 lse.data_ptr<float>(), B, Hq, Hkv, L, D, /*kv_stride=*/L,
                                                 n_.data_ptr<int32_t>(), window, (float)scale, num_splits,
                                                 ws.data_ptr(), ws_bytes, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gqaDecodeVarlen", rc);
        return pair_result(std::move(o), std::move(lse));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// decodeRopeAppend {B Hq Hkv L D} q kNew vNew cos sin kCache vCache pos stream : IO (T #[B,Hq,1,D])
// The caches are mutated in place (row `pos`), like the output tensors of the reference's launchers.
lean_object* lean_tyr_gpu_decode_rope_append(uint64_t B, uint64_t Hq, uint64_t Hkv, uint64_t L, uint64_t D,
                                             b_lean_obj_arg q, b_lean_obj_arg k_new, b_lean_obj_arg v_new,
                                             b_lean_obj_arg cos, b_lean_obj_arg sin, b_lean_obj_arg k_cache,
                                             b_lean_obj_arg v_cache, uint64_t pos, uint64_t stream,
                                             lean_object* /*world*/) {
    try {
        auto q_ = borrowTensor(q), kn = borrowTensor(k_new), vn = borrowTensor(v_new);
        auto c_ = borrowTensor(cos), s_ = borrowTensor(sin), kc = borrowTensor(k_cache), vc = borrowTensor(v_cache);
        std::string err;
        if (!check(q_, "q", torch::kBFloat16, err) || !check(kn, "kNew", torch::kBFloat16, err) ||
            !check(vn, "vNew", torch::kBFloat16, err) || !check(c_, "cos", torch::kFloat32, err) ||
            !check(s_, "sin", torch::kFloat32, err) || !check(kc, "kCache", torch::kBFloat16, err) ||
            !check(vc, "vCache", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, q_);   // outputs and scratch belong to the launch stream
        auto q_out = torch::empty_like(q_);
        const int rc = tyr_hip_decode_rope_append(q_.data_ptr(), kn.data_ptr(), vn.data_ptr(), c_.data_ptr<float>(),
                                                  s_.data_ptr<float>(), q_out.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                                  B, Hq, Hkv, D, L, pos, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("decodeRopeAppend", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(q_out)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// applyRotaryEmb {B S H D} x cos sin stream : IO (T #[B,S,H,D])
lean_object* lean_tyr_gpu_rope_fwd(uint64_t B, uint64_t S, uint64_t H, uint64_t D, b_lean_obj_arg x,
                                   b_lean_obj_arg cos, b_lean_obj_arg sin, uint64_t stream, lean_object* /*world*/) {
    try {
        auto x_ = borrowTensor(x), c_ = borrowTensor(cos), s_ = borrowTensor(sin);
        std::string err;
        const bool bf16 = x_.scalar_type() == torch::kBFloat16;
        if (!check(x_, "x", bf16 ? torch::kBFloat16 : torch::kFloat32, err) ||
            !check(c_, "cos", torch::kFloat32, err) || !check(s_, "sin", torch::kFloat32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, x_);   // outputs and scratch belong to the launch stream
        auto y = torch::empty_like(x_);
        const int rc = tyr_hip_rope_fwd(x_.data_ptr(), c_.data_ptr<float>(), s_.data_ptr<float>(), y.data_ptr(), B, S,
                                        H, D, bf16 ? TYR_HIP_BF16 : TYR_HIP_F32, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("applyRotaryEmb", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(y)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// fusedLayerNormResidual {rows d} x residual weight bias eps stream : IO (out x outResid)
lean_object* lean_tyr_gpu_layernorm_residual(uint64_t rows, uint64_t d, b_lean_obj_arg x, b_lean_obj_arg residual,
                                             b_lean_obj_arg weight, b_lean_obj_arg bias, double eps, uint64_t stream,
                                             lean_object* /*world*/) {
    try {
        auto x_ = borrowTensor(x), r_ = borrowTensor(residual), w_ = borrowTensor(weight), b_ = borrowTensor(bias);
        std::string err;
        if (!check(x_, "x", torch::kBFloat16, err) || !check(r_, "residual", torch::kBFloat16, err) ||
            !check(w_, "weight", torch::kBFloat16, err) || !check(b_, "bias", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, x_);   // outputs and scratch belong to the launch stream
        auto out = torch::empty_like(x_), out_resid = torch::empty_like(x_);
        const int rc = tyr_hip_layernorm_residual(x_.data_ptr(), r_.data_ptr(), w_.data_ptr(), b_.data_ptr(),
                                                  out.data_ptr(), out_resid.data_ptr(), rows, d, (float)eps,
                                                  reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("fusedLayerNormResidual", rc);
        return pair_result(std::move(out), std::move(out_resid));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// copy {s} input stream : IO (T s)      (the erased shape argument arrives as an owned object and is ignored)
lean_object* lean_tyr_gpu_copy(lean_obj_arg /*shape*/, b_lean_obj_arg input, uint64_t stream, lean_object* /*world*/) {
    try {
        auto in_ = borrowTensor(input);
        if (!in_.is_cuda()) return io_error("input must be a CUDA tensor");
        if (!in_.is_contiguous()) return io_error("input must be contiguous");
        LaunchStreamScope on_stream(stream, in_);   // outputs and scratch belong to the launch stream
        auto out = torch::empty_like(in_);
        const int rc = tyr_hip_copy(in_.data_ptr(), out.data_ptr(), (size_t)in_.nbytes(), reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("copy", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(out)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gemmBf16 {M N K} a b stream : IO (T #[M,N])
lean_object* lean_tyr_gpu_gemm_bf16(uint64_t M, uint64_t N, uint64_t K, b_lean_obj_arg a,
                                    b_lean_obj_arg b, uint64_t stream, lean_object* /*world*/) {
    try {
        auto a_ = borrowTensor(a), b_ = borrowTensor(b);
        std::string err;
        if (!check(a_, "a", torch::kBFloat16, err) || !check(b_, "b", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, a_);   // outputs and scratch belong to the launch stream
        auto c = torch::empty({(int64_t)M, (int64_t)N}, a_.options());
        const int rc = tyr_hip_gemm_bf16(a_.data_ptr(), b_.data_ptr(), c.data_ptr(), M, N, K, 0,
                                         reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gemmBf16", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(c)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gemmBf16NT {M N K} a (b : T #[N,K]) stream : IO (T #[M,N])   -- the N x K form of tiledAccumulator
lean_object* lean_tyr_gpu_gemm_bf16_nt(uint64_t M, uint64_t N, uint64_t K, b_lean_obj_arg a,
                                       b_lean_obj_arg b, uint64_t stream, lean_object* /*world*/) {
    try {
        auto a_ = borrowTensor(a), b_ = borrowTensor(b);
        std::string err;
        if (!check(a_, "a", torch::kBFloat16, err) || !check(b_, "b", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, a_);   // outputs and scratch belong to the launch stream
        auto c = torch::empty({(int64_t)M, (int64_t)N}, a_.options());
        const int rc = tyr_hip_gemm_bf16(a_.data_ptr(), b_.data_ptr(), c.data_ptr(), M, N, K, 1,
                                         reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gemmBf16NT", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(c)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gemmFp8 {M N K} a b scaleA scaleB stream : IO (T #[M,N])
lean_object* lean_tyr_gpu_gemm_fp8(uint64_t M, uint64_t N, uint64_t K, b_lean_obj_arg a,
                                   b_lean_obj_arg b, double scale_a, double scale_b, uint64_t stream,
                                   lean_object* /*world*/) {
    try {
        auto a_ = borrowTensor(a), b_ = borrowTensor(b);
        std::string err;
        if (!check(a_, "a", torch::kFloat8_e4m3fn, err) || !check(b_, "b", torch::kFloat8_e4m3fn, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, a_);   // outputs and scratch belong to the launch stream
        auto c = torch::empty({(int64_t)M, (int64_t)N}, a_.options().dtype(torch::kBFloat16));
        const int rc = tyr_hip_gemm_fp8(a_.data_ptr(), b_.data_ptr(), c.data_ptr(), M, N, K, (float)scale_a,
                                        (float)scale_b, 0, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gemmFp8", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(c)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// matmulBf16 {Bt M N K} a b stream : IO (T #[Bt,M,N])   -- `lean_torch_matmul` on rank-3 operands, one launch
lean_object* lean_tyr_gpu_matmul_bf16(uint64_t Bt, uint64_t M, uint64_t N, uint64_t K, b_lean_obj_arg a,
                                      b_lean_obj_arg b, uint64_t stream, lean_object* /*world*/) {
    try {
        auto a_ = borrowTensor(a), b_ = borrowTensor(b);
        std::string err;
        if (!check(a_, "a", torch::kBFloat16, err) || !check(b_, "b", torch::kBFloat16, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, a_);   // outputs and scratch belong to the launch stream
        auto c = torch::empty({(int64_t)Bt, (int64_t)M, (int64_t)N}, a_.options());
        const int rc = tyr_hip_gemm_bf16_batched(a_.data_ptr(), b_.data_ptr(), c.data_ptr(), Bt, M, N, K, M * K, K * N,
                                                 M * N, 0, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("matmulBf16", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(c)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gemmFp8Scaled {M N K} a b rowScale colScale stream : IO (T #[M,N])   -- f32 out, per-row x per-column scales
lean_object* lean_tyr_gpu_gemm_fp8_scaled(uint64_t M, uint64_t N, uint64_t K, b_lean_obj_arg a, b_lean_obj_arg b,
                                          b_lean_obj_arg row_scale, b_lean_obj_arg col_scale, uint64_t stream,
                                          lean_object* /*world*/) {
    try {
        auto a_ = borrowTensor(a), b_ = borrowTensor(b), r_ = borrowTensor(row_scale), c_ = borrowTensor(col_scale);
        std::string err;
        if (!check(a_, "a", torch::kFloat8_e4m3fn, err) || !check(b_, "b", torch::kFloat8_e4m3fn, err) ||
            !check(r_, "rowScale", torch::kFloat32, err) || !check(c_, "colScale", torch::kFloat32, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, a_);   // outputs and scratch belong to the launch stream
        auto c = torch::empty({(int64_t)M, (int64_t)N}, a_.options().dtype(torch::kFloat32));
        const int rc = tyr_hip_gemm_fp8_ex(a_.data_ptr(), b_.data_ptr(), c.data_ptr(), M, N, K, 1.0f, r_.data_ptr<float>(),
                                           c_.data_ptr<float>(), TYR_HIP_OUT_F32, 0, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gemmFp8Scaled", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(c)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// gemmFp8E4M3 {M N K} a b scale stream : IO (T #[M,N])   -- E4M3 out (tkH100Fp8E4M3GemmFwd)
lean_object* lean_tyr_gpu_gemm_fp8_e4m3(uint64_t M, uint64_t N, uint64_t K, b_lean_obj_arg a, b_lean_obj_arg b,
                                        double scale, uint64_t stream, lean_object* /*world*/) {
    try {
        auto a_ = borrowTensor(a), b_ = borrowTensor(b);
        std::string err;
        if (!check(a_, "a", torch::kFloat8_e4m3fn, err) || !check(b_, "b", torch::kFloat8_e4m3fn, err))
            return io_error(err);
        LaunchStreamScope on_stream(stream, a_);   // outputs and scratch belong to the launch stream
        auto c = torch::empty({(int64_t)M, (int64_t)N}, a_.options());
        const int rc = tyr_hip_gemm_fp8_ex(a_.data_ptr(), b_.data_ptr(), c.data_ptr(), M, N, K, (float)scale, nullptr,
                                           nullptr, TYR_HIP_OUT_E4M3, 0, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("gemmFp8E4M3", rc);
        return lean_io_result_mk_ok(giveTensor(std::move(c)));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// lossAndGradOut {s} out target stream : IO (T #[] x T s)   -- loss = 0.5 mean((out - target)^2), dO = bf16((out - target) / n)
lean_object* lean_tyr_gpu_mse_loss_grad(lean_obj_arg /*shape*/, b_lean_obj_arg out, b_lean_obj_arg target, uint64_t stream,
                                        lean_object* /*world*/) {
    try {
        auto o_ = borrowTensor(out), t_ = borrowTensor(target);
        std::string err;
        if (!check(o_, "out", torch::kBFloat16, err) || !check(t_, "target", torch::kBFloat16, err)) return io_error(err);
        if (o_.numel() != t_.numel()) return io_error("out and target must have the same shape");
        LaunchStreamScope on_stream(stream, o_);   // outputs and scratch belong to the launch stream
        auto d_o = torch::empty_like(o_);
        auto loss = torch::empty({}, o_.options().dtype(torch::kFloat32));
        const size_t ws_bytes = tyr_hip_mse_loss_grad_workspace_bytes((uint64_t)o_.numel());
        auto ws = torch::empty({(int64_t)(ws_bytes ? ws_bytes : 16)}, o_.options().dtype(torch::kUInt8));
        const int rc = tyr_hip_mse_loss_grad(o_.data_ptr(), t_.data_ptr(), d_o.data_ptr(), loss.data_ptr<float>(),
                                             (uint64_t)o_.numel(), ws.data_ptr(), ws_bytes, reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("lossAndGradOut", rc);
        return pair_result(std::move(loss), std::move(d_o));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

// sgdUpdate {s} param grad lr stream : IO (T s x T s)   -- (param - f32(grad) * lr, its bf16 copy)
lean_object* lean_tyr_gpu_sgd_step(lean_obj_arg /*shape*/, b_lean_obj_arg param, b_lean_obj_arg grad, double lr,
                                   uint64_t stream, lean_object* /*world*/) {
    try {
        auto p_ = borrowTensor(param), g_ = borrowTensor(grad);
        std::string err;
        if (!check(p_, "param", torch::kFloat32, err) || !check(g_, "grad", torch::kBFloat16, err)) return io_error(err);
        if (p_.numel() != g_.numel()) return io_error("param and grad must have the same shape");
        LaunchStreamScope on_stream(stream, p_);   // outputs and scratch belong to the launch stream
        auto p_new = torch::empty_like(p_);
        auto p_low = torch::empty_like(g_);
        const int rc = tyr_hip_sgd_step(p_.data_ptr<float>(), g_.data_ptr(), (float)lr, p_new.data_ptr<float>(), p_low.data_ptr(),
                                        (uint64_t)p_.numel(), reinterpret_cast<void*>(stream));
        if (rc != TYR_HIP_OK) return status_error("sgdUpdate", rc);
        return pair_result(std::move(p_new), std::move(p_low));
    } catch (const std::exception& e) {
        return io_error(e.what());
    }
}

}  // extern "C"
#endif  // TYR_HAVE_LEAN
