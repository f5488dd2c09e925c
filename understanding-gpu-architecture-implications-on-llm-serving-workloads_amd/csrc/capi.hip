// C ABI of libmi355_serving.so (see include/mi355_serving.h): argument validation and error reporting around
// the kernel dispatchers. Nothing here allocates device memory or synchronises.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include "mi355_serving_internal.h"

namespace {
thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}
int hip_fail(hipError_t e, const char* what) {
    return fail(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}
}  // namespace

extern "C" {

int mi355_hgemm(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                int layout, void* stream) {
    if (!A || !B || !C) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_hgemm: null pointer");
    if (M < 1 || N < 1 || K < 1) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_hgemm: M, N, K must be >= 1 (got %d, %d, %d)", M, N, K);
    if (layout != MI355_GEMM_NN && layout != MI355_GEMM_NT && layout != MI355_GEMM_TN)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_hgemm: unknown layout %d", layout);
    const int64_t a_min = (layout == MI355_GEMM_TN) ? M : K;
    const int64_t b_min = (layout == MI355_GEMM_NT) ? K : N;
    if (lda < a_min || ldb < b_min || ldc < N)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_hgemm: leading dimension too small (lda %lld >= %lld, ldb %lld >= %lld, ldc %lld >= %d required)",
                    (long long)lda, (long long)a_min, (long long)ldb, (long long)b_min, (long long)ldc, N);
    hipError_t e = mi355::hgemm_dispatch(A, B, C, M, N, K, lda, ldb, ldc, layout, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "mi355_hgemm launch");
    return 0;
}

int mi355_fmha_fwd(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                   int Sk, int D, float scale, int causal, int kv_valid_len, void* stream) {
    if (!Q || !K || !V || !O) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd: null pointer");
    if (B < 1 || Hq < 1 || Hkv < 1 || Sq < 1 || Sk < 1)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd: B, Hq, Hkv, Sq, Sk must be >= 1");
    if (D != 128) return fail(MI355_ERR_UNSUPPORTED, "mi355_fmha_fwd: head_dim must be 128 (got %d)", D);
    if (Hq % Hkv != 0) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd: Hq (%d) must be a multiple of Hkv (%d)", Hq, Hkv);
    if (kv_valid_len < 1 || kv_valid_len > Sk)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd: kv_valid_len %d outside [1, Sk=%d]", kv_valid_len, Sk);
    if (!(scale > 0.f) || scale > 3.0e38f)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd: scale must be positive and finite (got %g)", (double)scale);
    if ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(V) |
         reinterpret_cast<uintptr_t>(O)) % 16 != 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd: Q, K, V, O must be 16-byte aligned");
    hipError_t e = mi355::fmha_fwd_dispatch(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale, causal != 0, kv_valid_len,
                                            static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "mi355_fmha_fwd launch");
    return 0;
}

const char* mi355_last_error(void) { return g_err; }

int mi355_serving_version(void) { return MI355_SERVING_VERSION; }

}  // extern "C"
