// PyTorch operator layer of fmha_unified for MI355X.
//
// Same operator surface as the reference (kernels/fmha/pkg/fmha_unified/csrc/fmha_kernel.cpp:9-18): schemas
// `fmha_unified::finefmha_0 .. finefmha_7 (Tensor q, Tensor k, Tensor v, bool causal, bool is_decode,
// int decode_length) -> Tensor`, CUDA dispatch key, empty `_C` module. Every index runs the one gfx950
// attention kernel of libmi355_serving.so, for float16 or bfloat16 tensors. Host checks mirror
// semi/fmha_2_amd.cpp:322-333 (dtype, d == 128,
// is_decode implies !causal) and add the shape checks the reference omits.
//
// One operator is added without touching the reference's schemas:
//   `finefmha_fwd_lse(q, k, v, causal, is_decode, decode_length) -> (Tensor out, Tensor lse)`
// which also returns the log-sum-exp [B, Hq, Sq] in fp32 (the reference has no LSE output).
//
// decode_length is the number of valid keys (ops.py:18 passes the un-padded k.size(2)); keys at or beyond it
// are masked. The reference masks `k > decode_length` (fmha_2_amd.cpp:191), which lets the first padded key
// through; that off-by-one is not reproduced.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <cmath>
#include <tuple>

#include "mi355_serving.h"

namespace fmha_unified {

// Registers _C as a Python extension module.
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {}

namespace {

// A [B, H, S, D] view the kernels can read in place: contiguous last dimension, every other stride a non-negative
// multiple of 8 elements, 16-byte aligned base. This covers `x.view(B, S, H, D).transpose(1, 2)` and slices of a fused
// QKV projection, the forms the reference's in-model caller produces (benchmarks/flashattn-cuda/modeling_llama.py:658-660)
// and which kernels/fmha/pkg/fmha_unified/ops.py:23-25 copies into contiguous tensors first.
bool readable_in_place(const at::Tensor& t) {
    if (t.stride(3) != 1 || reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 != 0) return false;
    for (int i = 0; i < 3; ++i)
        if (t.stride(i) < 0 || t.stride(i) % 8 != 0) return false;
    return true;
}

std::tuple<at::Tensor, at::Tensor> run_fmha(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, bool causal,
                                            bool is_decode, int64_t decode_length, bool want_lse) {
    const char* name = "finefmha";
    TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, name, ": q, k, v must be [B, H, S, D] tensors");
    const bool bf16 = q.scalar_type() == at::kBFloat16;  // the dtype of the reference's finefmha_5 (manual/fmha_5_nv.cu:148-150)
    TORCH_CHECK(q.scalar_type() == at::kHalf || bf16, name, ": q must be float16 or bfloat16, got ", q.scalar_type());
    TORCH_CHECK(k.scalar_type() == q.scalar_type(), name, ": k must have q's dtype ", q.scalar_type(), ", got ", k.scalar_type());
    TORCH_CHECK(v.scalar_type() == q.scalar_type(), name, ": v must have q's dtype ", q.scalar_type(), ", got ", v.scalar_type());
    const int64_t B = q.size(0), Hq = q.size(1), Sq = q.size(2), D = q.size(3);
    const int64_t Hkv = k.size(1), Sk = k.size(2);
    TORCH_CHECK(D == 128, name, ": head embedding dimension must be 128, got ", D);
    TORCH_CHECK(k.size(0) == B && k.size(3) == D, name, ": k shape does not match q");
    TORCH_CHECK(v.sizes() == k.sizes(), name, ": v shape must equal k shape");
    TORCH_CHECK(B >= 1 && Hq >= 1 && Hkv >= 1 && Sq >= 1 && Sk >= 1, name, ": empty tensors are not supported");
    TORCH_CHECK(Hq % Hkv == 0, name, ": number of q heads (", Hq, ") must be a multiple of kv heads (", Hkv, ")");
    TORCH_CHECK(!(is_decode && causal), name, ": causal is not supported in decode mode");
    TORCH_CHECK(decode_length >= 1 && decode_length <= Sk, name, ": decode_length ", decode_length,
                " outside [1, k.size(2) = ", Sk, "]");
    TORCH_CHECK(Sq <= INT32_MAX && Sk <= INT32_MAX && B <= INT32_MAX && Hq <= INT32_MAX, name, ": dimension exceeds int32");
    TORCH_CHECK(q.is_cuda() && k.is_cuda() && v.is_cuda(), name, ": q, k, v must be GPU tensors");
    TORCH_CHECK(q.device() == k.device() && q.device() == v.device(), name, ": q, k, v are on different devices");

    // torch on ROCm presents HIP devices under the "cuda" device type; these are its guard and stream for them
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    at::Tensor qc = readable_in_place(q) ? q : q.contiguous();
    at::Tensor kc = readable_in_place(k) ? k : k.contiguous();
    at::Tensor vc = readable_in_place(v) ? v : v.contiguous();
    // The result is a freshly allocated contiguous [B, H, S, D] tensor whatever the strides of q, as in the reference
    // (`zeros_like` of a `.contiguous()` input, semi/fmha_2_amd.cpp:336; kernels/fmha/pkg/fmha_unified/ops.py:23-29), so
    // callers may `.view()` it. empty() instead of zeros(): the kernel writes every element.
    at::Tensor o = at::empty(qc.sizes(), qc.options());
    at::Tensor lse;
    float* lse_ptr = nullptr;
    if (want_lse) {
        lse = at::empty({B, Hq, Sq}, qc.options().dtype(at::kFloat));
        lse_ptr = lse.data_ptr<float>();
    }
    const float scale = 1.0f / std::sqrt(static_cast<float>(D));  // fmha_2_amd.cpp:320
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    const int64_t strides[12] = {qc.stride(0), qc.stride(1), qc.stride(2), kc.stride(0), kc.stride(1), kc.stride(2),
                                 vc.stride(0), vc.stride(1), vc.stride(2), o.stride(0),  o.stride(1),  o.stride(2)};
    auto entry = bf16 ? &mi355_fmha_fwd_bf16 : &mi355_fmha_fwd_strided;
    int rc = entry(qc.data_ptr(), kc.data_ptr(), vc.data_ptr(), o.data_ptr(), lse_ptr, (int)B, (int)Hq, (int)Hkv, (int)Sq,
                   (int)Sk, (int)D, scale, causal ? 1 : 0, (int)decode_length, strides, stream);
    TORCH_CHECK(rc == 0, name, ": ", mi355_last_error(), " (code ", rc, ")");
    return {o, lse};
}

at::Tensor finefmha(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, bool causal, bool is_decode,
                    int64_t decode_length) {
    return std::get<0>(run_fmha(q, k, v, causal, is_decode, decode_length, false));
}

std::tuple<at::Tensor, at::Tensor> finefmha_fwd_lse(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                                    bool causal, bool is_decode, int64_t decode_length) {
    return run_fmha(q, k, v, causal, is_decode, decode_length, true);
}

}  // namespace

// Defines the operators (the first eight schema strings are the reference's).
TORCH_LIBRARY(fmha_unified, m) {
    m.def("finefmha_0(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_1(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_2(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_3(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_4(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_5(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_6(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_7(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> Tensor");
    m.def("finefmha_fwd_lse(Tensor q, Tensor k, Tensor v, bool causal, bool is_decode, int decode_length) -> (Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(fmha_unified, CUDA, m) {
    m.impl("finefmha_0", &finefmha);
    m.impl("finefmha_1", &finefmha);
    m.impl("finefmha_2", &finefmha);
    m.impl("finefmha_3", &finefmha);
    m.impl("finefmha_4", &finefmha);
    m.impl("finefmha_5", &finefmha);
    m.impl("finefmha_6", &finefmha);
    m.impl("finefmha_7", &finefmha);
    m.impl("finefmha_fwd_lse", &finefmha_fwd_lse);
}

// The same functions under the CPU key: CPU tensors then reach the argument validation above and are
// rejected with its message ("must be GPU tensors") instead of a dispatcher error. Nothing is computed on the CPU.
TORCH_LIBRARY_IMPL(fmha_unified, CPU, m) {
    m.impl("finefmha_0", &finefmha);
    m.impl("finefmha_1", &finefmha);
    m.impl("finefmha_2", &finefmha);
    m.impl("finefmha_3", &finefmha);
    m.impl("finefmha_4", &finefmha);
    m.impl("finefmha_5", &finefmha);
    m.impl("finefmha_6", &finefmha);
    m.impl("finefmha_7", &finefmha);
    m.impl("finefmha_fwd_lse", &finefmha_fwd_lse);
}

}  // namespace fmha_unified
