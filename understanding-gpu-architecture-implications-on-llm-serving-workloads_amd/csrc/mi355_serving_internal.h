// Internal C++ entry points behind the C ABI of include/mi355_serving.h.
#pragma once
#include <hip/hip_runtime.h>
#include "../../include/mi355_serving.h"

namespace mi355 {

// Launches the GEMM kernels; arguments as mi355_hgemm after validation.
hipError_t hgemm_dispatch(const void* A, const void* B, void* C, int M, int N, int K, long lda, long ldb, long ldc,
                          int layout, hipStream_t stream);

// Element strides of the attention operands: tensor[b][h][s][d] lives at b*batch + h*head + s*row + d (d contiguous).
struct FmhaStrides {
    long q_batch, q_head, q_row;
    long k_batch, k_head, k_row;
    long v_batch, v_head, v_row;
    long o_batch, o_head, o_row;
};

// Launches the attention forward kernels; arguments as mi355_fmha_fwd_strided after validation.
hipError_t fmha_fwd_dispatch(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                             int Sq, int Sk, float scale, int causal, int kv_valid_len, const FmhaStrides& strides,
                             hipStream_t stream);

// Split-KV path for few query rows per kv head (generation step); see fmha_decode.hip.
bool fmha_decode_applicable(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len);
hipError_t fmha_decode_dispatch(const _Float16* Q, const _Float16* K, const _Float16* V, _Float16* O, float* LSE, int B, int Hq,
                                int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid_len, const FmhaStrides& strides,
                                hipStream_t stream);

}  // namespace mi355
