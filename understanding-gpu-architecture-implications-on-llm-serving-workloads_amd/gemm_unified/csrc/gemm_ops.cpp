// PyTorch operator layer of gemm_unified for MI355X.
//
// Same operator surface as the reference (kernels/gemm/pkg/gemm_unified/csrc/gemm_kernel.cpp:9-27): schemas
// `gemm_unified::finegemm_0 .. finegemm_16 (Tensor a, Tensor b) -> Tensor`, implementations registered under
// the CUDA dispatch key (the key HIP tensors use), and an empty `_C` python module whose import runs the
// registrars (gemm_kernel.cpp:6). Every index is backed by the one gfx950 kernel family in libmi355_serving.so;
// what differs per index is only the operand layout the reference's kernels of that index read
// (kernels/gemm/test/correct.py:9-15):
//     0..11   C = a[M,K]   * b[K,N]
//     12, 16  C = a[K,M]^T * b[K,N]     (manual/gemm_12_amd.cpp:52-57, manual/gemm_16_amd.cpp:55-57)
//     13..15  C = a[M,K]   * b[N,K]^T   (manual/gemm_13_amd.cpp:58-60)
// Unlike the reference wrappers (manual/gemm_16_amd.cpp:345-367) the shapes are taken from the true layout, so
// non-square operands work, the output is allocated with empty() instead of zeros(), the launch goes to the
// current stream, and every argument is validated before the device is touched.
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include "mi355_serving.h"

namespace gemm_unified {

// Registers _C as a Python extension module.
PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {}

namespace {

at::Tensor run_gemm(const at::Tensor& a, const at::Tensor& b, int layout, const char* name) {
    TORCH_CHECK(a.dim() == 2 && b.dim() == 2, name, ": a and b must be 2-D, got ", a.dim(), "-D and ", b.dim(), "-D");
    const bool bf16 = a.scalar_type() == at::kBFloat16;
    TORCH_CHECK(a.scalar_type() == at::kHalf || bf16, name, ": a must be float16 or bfloat16, got ", a.scalar_type());
    TORCH_CHECK(b.scalar_type() == a.scalar_type(), name, ": b must have a's dtype ", a.scalar_type(), ", got ", b.scalar_type());
    int64_t M, N, K, Kb;
    if (layout == MI355_GEMM_TN) {
        K = a.size(0); M = a.size(1);
    } else {
        M = a.size(0); K = a.size(1);
    }
    if (layout == MI355_GEMM_NT) {
        N = b.size(0); Kb = b.size(1);
    } else {
        Kb = b.size(0); N = b.size(1);
    }
    TORCH_CHECK(K == Kb, name, ": inner dimensions differ (", K, " vs ", Kb, ")");
    TORCH_CHECK(M >= 1 && N >= 1 && K >= 1, name, ": empty operands are not supported");
    TORCH_CHECK(M <= INT32_MAX && N <= INT32_MAX && K <= INT32_MAX, name, ": dimension exceeds int32");
    TORCH_CHECK(a.is_cuda() && b.is_cuda(), name, ": a and b must be GPU tensors");
    TORCH_CHECK(a.device() == b.device(), name, ": a and b are on different devices");

    // torch on ROCm presents HIP devices under the "cuda" device type; these are its guard and stream for them
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
    at::Tensor ac = a.contiguous();
    at::Tensor bc = b.contiguous();
    at::Tensor c = at::empty({M, N}, a.options());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
    auto entry = bf16 ? &mi355_gemm_bf16 : &mi355_hgemm;
    // Leading dimensions are the logical row lengths of the contiguous operands, not stride(0): torch ignores the stride of
    // a size-1 dimension when it decides contiguity, so a [1, K] operand may carry any stride(0).
    const int64_t lda = ac.size(1), ldb = bc.size(1);
    int rc = entry(ac.data_ptr(), bc.data_ptr(), c.data_ptr(), (int)M, (int)N, (int)K, lda, ldb, N, layout, stream);
    TORCH_CHECK(rc == 0, name, ": ", mi355_last_error(), " (code ", rc, ")");
    return c;
}

template <int LAYOUT>
at::Tensor finegemm(const at::Tensor& a, const at::Tensor& b) {
    return run_gemm(a, b, LAYOUT, "finegemm");
}

}  // namespace

// Defines the operators (same schema strings as the reference).
TORCH_LIBRARY(gemm_unified, m) {
    m.def("finegemm_0(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_1(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_2(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_3(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_4(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_5(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_6(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_7(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_8(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_9(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_10(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_11(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_12(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_13(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_14(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_15(Tensor a, Tensor b) -> Tensor");
    m.def("finegemm_16(Tensor a, Tensor b) -> Tensor");
}

// One implementation per schema name; HIP tensors dispatch on the CUDA key.
TORCH_LIBRARY_IMPL(gemm_unified, CUDA, m) {
    m.impl("finegemm_0", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_1", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_2", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_3", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_4", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_5", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_6", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_7", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_8", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_9", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_10", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_11", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_12", &finegemm<MI355_GEMM_TN>);
    m.impl("finegemm_13", &finegemm<MI355_GEMM_NT>);
    m.impl("finegemm_14", &finegemm<MI355_GEMM_NT>);
    m.impl("finegemm_15", &finegemm<MI355_GEMM_NT>);
    m.impl("finegemm_16", &finegemm<MI355_GEMM_TN>);
}

// The same functions under the CPU key: CPU tensors then reach the argument validation above and are
// rejected with its message ("must be GPU tensors") instead of a dispatcher error. Nothing is computed on the CPU.
TORCH_LIBRARY_IMPL(gemm_unified, CPU, m) {
    m.impl("finegemm_0", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_1", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_2", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_3", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_4", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_5", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_6", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_7", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_8", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_9", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_10", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_11", &finegemm<MI355_GEMM_NN>);
    m.impl("finegemm_12", &finegemm<MI355_GEMM_TN>);
    m.impl("finegemm_13", &finegemm<MI355_GEMM_NT>);
    m.impl("finegemm_14", &finegemm<MI355_GEMM_NT>);
    m.impl("finegemm_15", &finegemm<MI355_GEMM_NT>);
    m.impl("finegemm_16", &finegemm<MI355_GEMM_TN>);
}

}  // namespace gemm_unified
