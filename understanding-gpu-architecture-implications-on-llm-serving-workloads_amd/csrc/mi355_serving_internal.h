// Internal C++ entry points behind the C ABI of include/mi355_serving.h.
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include <cstddef>
#include "../../include/mi355_serving.h"

namespace mi355 {

// Raises a kernel's dynamic LDS limit once per device (the attribute belongs to the device the call is made on).
// Threads may race to set it; the call is idempotent, so the flags only need to be atomic.
struct DynamicLdsOnce {
    static constexpr int kMaxDevices = 64;
    std::atomic<bool> done[kMaxDevices] = {};
    hipError_t ensure(const void* kernel, int bytes) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const bool tracked = dev >= 0 && dev < kMaxDevices;
        if (tracked && done[dev].load(std::memory_order_acquire)) return hipSuccess;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e == hipSuccess && tracked) done[dev].store(true, std::memory_order_release);
        return e;
    }
};

// Launches the GEMM kernels; arguments as mi355_hgemm_add after validation (R == nullptr: no residual).
// `variant` pins a tile shape instead of the choice by shape (0); see mi355_internal_hgemm_variant below.
hipError_t hgemm_dispatch(const void* A, const void* B, void* C, const void* R, int M, int N, int K, long lda, long ldb,
                          long ldc, long ldr, int layout, int dtype, int variant, hipStream_t stream);

// Element strides of the attention operands: tensor[b][h][s][d] lives at b*batch + h*head + s*row + d (d contiguous).
struct FmhaStrides {
    long q_batch, q_head, q_row;
    long k_batch, k_head, k_row;
    long v_batch, v_head, v_row;
    long o_batch, o_head, o_row;
};

// The product fused with silu(gate) * up (see hgemm_main_kernel's EPI); hipErrorNotSupported for shapes without it.
hipError_t hgemm_silu_mul_dispatch(const void* A, const void* B, void* C, int M, int N2, int K, long lda, long ldb, long ldc,
                                   int layout, int dtype, hipStream_t stream);

// Where the split-KV and key-range attention paths keep their partial results.
struct FmhaWorkspace {
    enum Kind { kLibrary, kCaller, kStatic };
    Kind kind = kLibrary;     // kLibrary: the library's own grow-only buffer of (device, stream)
    void* ptr = nullptr;      // kCaller: device memory of the caller, `bytes` long
    size_t bytes = 0;         // kStatic: the fixed-size __device__ array of fmha_decode.hip (nothing is ever allocated)
};

// Launches the attention forward kernels; arguments as mi355_fmha_fwd_strided after validation.
// `variant` pins a kernel instead of the choice by shape (0); see mi355_internal_fmha_fwd_variant below.
hipError_t fmha_fwd_dispatch(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                             int Sq, int Sk, float scale, int causal, int kv_valid_len, const FmhaStrides& strides,
                             int dtype, int variant, const FmhaWorkspace& ws, hipStream_t stream);

// Split-KV path for few query rows per kv head (generation step); see fmha_decode.hip.
bool fmha_decode_applicable(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len);
// Bytes of workspace a call with these sizes uses (0 when it does not take the split-KV path).
size_t fmha_decode_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len);
// Bytes of workspace the key-range path of fmha_fwd.hip uses for a call with these sizes (0 when it does not take it), and
// the bytes a call uses on whichever of the two paths it takes.
size_t fmha_key_range_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len);
size_t fmha_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len);
// Size of the static scratch array behind FmhaWorkspace::kStatic.
size_t fmha_decode_static_scratch_bytes();
template <typename T>
hipError_t fmha_decode_dispatch(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq, int Hkv, int Sq, int Sk,
                                float scale, int causal, int kv_valid_len, const FmhaStrides& strides, const FmhaWorkspace& ws,
                                hipStream_t stream);

// Layer glue (glue.hip); arguments as the mi355_rmsnorm / mi355_rope / mi355_silu_mul entry points after validation.
hipError_t rmsnorm_dispatch(const void* x, const void* residual, void* res_out, const void* weight, void* out, long rows,
                            int hidden, long ldx, long ldr, long ldro, long ldo, float eps, int dtype, hipStream_t stream);
// rope_dispatch: `heads` heads are rotated, the first `inplace_heads` of them in place, `copy_heads` more are copied;
// consecutive heads of `out` lie o_head elements apart.
hipError_t rope_dispatch(const void* x, void* out, int B, int S, int inplace_heads, int heads, int copy_heads, long x_batch,
                         long x_row, long o_batch, long o_row, long o_head, const float* cos_t, const float* sin_t, const int* positions, long pos_batch,
                         int n_pos, int dtype, hipStream_t stream);
hipError_t silu_mul_dispatch(const void* in, void* out, long rows, int inter, int block, long ld_in, long ld_out, int dtype,
                             hipStream_t stream);

}  // namespace mi355

// Test and tuning hooks: exported from the shared library but not part of its public header. They take the kernel
// variant as an argument (no process-wide state): variants that do not fit the shape fall back to the choice by shape.
//   gemm: 0 = by shape; 1 = 256x256 tiles, 2 = 128x128, 3 = 64x128 (layout NT: 128x64), 4 = 64x64 with a ring of four
//         stages, 5 = 128x256, 6 = 256x128, 7 = 32x64 (layouts NN and NT): the tiled kernel of that shape for any product the tiled kernels take (M and N need not be multiples
//         of the tile); products of up to 64 rows that the small-M kernels take stay on those
//   fmha: 0 = by shape, 1 = 128-query workgroups, 2 = 256-query workgroups (1 and 2 also keep generation-step shapes off
//         the split-KV path), 3 = keys cut into ranges and merged (an error where the choice by shape would not do that)
extern "C" {
int mi355_internal_hgemm_variant(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb,
                                 int64_t ldc, int layout, int dtype, int variant, void* stream);
int mi355_internal_fmha_fwd_variant(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                                    int Sq, int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides,
                                    int dtype, int variant, void* stream);
}
