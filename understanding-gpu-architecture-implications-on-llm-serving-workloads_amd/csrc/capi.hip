// C ABI of libmi355_serving.so (see include/mi355_serving.h): argument validation and error reporting around
// the kernel dispatchers. Nothing here allocates device memory or synchronises (the one allocation the library ever
// makes, the split-KV workspace of mi355_fmha_fwd*, lives in fmha_decode.hip).
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
mi355::FmhaStrides contiguous_strides(int Hq, int Hkv, int Sq, int Sk, int D) {
    const long q_head = (long)Sq * D, k_head = (long)Sk * D;
    return {Hq * q_head, q_head, D, Hkv * k_head, k_head, D, Hkv * k_head, k_head, D, Hq * q_head, q_head, D};
}
mi355::FmhaStrides strides_from(const int64_t* s) {
    return {(long)s[0], (long)s[1], (long)s[2], (long)s[3], (long)s[4], (long)s[5],
            (long)s[6], (long)s[7], (long)s[8], (long)s[9], (long)s[10], (long)s[11]};
}
}  // namespace

extern "C" {

// R == nullptr: the plain product; otherwise the residual operand of the *_add entry points (checked by the caller)
static int hgemm_impl(const char* fn, int dtype, const void* A, const void* B, void* C, const void* R, int M, int N, int K, int64_t lda,
                      int64_t ldb, int64_t ldc, int64_t ldr, int layout, void* stream, int variant = 0) {
    if (!A || !B || !C) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if (M < 1 || N < 1 || K < 1) return fail(MI355_ERR_BAD_ARGUMENT, "%s: M, N, K must be >= 1 (got %d, %d, %d)", fn, M, N, K);
    if (layout != MI355_GEMM_NN && layout != MI355_GEMM_NT && layout != MI355_GEMM_TN)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: unknown layout %d", fn, layout);
    const int64_t a_min = (layout == MI355_GEMM_TN) ? M : K;
    const int64_t b_min = (layout == MI355_GEMM_NT) ? K : N;
    if (lda < a_min || ldb < b_min || ldc < N)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: leading dimension too small (lda %lld >= %lld, ldb %lld >= %lld, ldc %lld >= %d required)", fn,
                    (long long)lda, (long long)a_min, (long long)ldb, (long long)b_min, (long long)ldc, N);
    if (R != nullptr && ldr < N)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: leading dimension too small (ldr %lld >= %d required)", fn, (long long)ldr, N);
    if (R != nullptr && R == C && ldr != ldc)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: R aliases C but ldr (%lld) differs from ldc (%lld)", fn, (long long)ldr, (long long)ldc);
    hipError_t e = mi355::hgemm_dispatch(A, B, C, R, M, N, K, lda, ldb, ldc, R ? ldr : 0, layout, dtype, variant, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

int mi355_hgemm(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                int layout, void* stream) {
    return hgemm_impl("mi355_hgemm", MI355_DTYPE_FP16, A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, layout, stream);
}

int mi355_gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                int layout, void* stream) {
    return hgemm_impl("mi355_gemm_bf16", MI355_DTYPE_BF16, A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, layout, stream);
}

int mi355_hgemm_add(const void* A, const void* B, const void* R, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldr,
                    int64_t ldc, int layout, void* stream) {
    if (!R) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_hgemm_add: null pointer");
    return hgemm_impl("mi355_hgemm_add", MI355_DTYPE_FP16, A, B, C, R, M, N, K, lda, ldb, ldc, ldr, layout, stream);
}

int mi355_gemm_add_bf16(const void* A, const void* B, const void* R, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldr,
                        int64_t ldc, int layout, void* stream) {
    if (!R) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_gemm_add_bf16: null pointer");
    return hgemm_impl("mi355_gemm_add_bf16", MI355_DTYPE_BF16, A, B, C, R, M, N, K, lda, ldb, ldc, ldr, layout, stream);
}


static int fmha_checked(const char* fn, const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                        int Sq, int Sk, int D, float scale, int causal, int kv_valid_len, const mi355::FmhaStrides& sd,
                        int dtype, void* stream, int variant = 0, const mi355::FmhaWorkspace& ws = mi355::FmhaWorkspace()) {
    if (!Q || !K || !V || !O) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if (B < 1 || Hq < 1 || Hkv < 1 || Sq < 1 || Sk < 1)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: B, Hq, Hkv, Sq, Sk must be >= 1", fn);
    if (D != 128) return fail(MI355_ERR_UNSUPPORTED, "%s: head_dim must be 128 (got %d)", fn, D);
    if (Hq % Hkv != 0) return fail(MI355_ERR_BAD_ARGUMENT, "%s: Hq (%d) must be a multiple of Hkv (%d)", fn, Hq, Hkv);
    if (kv_valid_len < 1 || kv_valid_len > Sk)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: kv_valid_len %d outside [1, Sk=%d]", fn, kv_valid_len, Sk);
    if (!(scale > 0.f) || scale > 3.0e38f)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: scale must be positive and finite (got %g)", fn, (double)scale);
    if ((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(V) |
         reinterpret_cast<uintptr_t>(O)) % 16 != 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: Q, K, V, O must be 16-byte aligned", fn);
    const long all[12] = {sd.q_batch, sd.q_head, sd.q_row, sd.k_batch, sd.k_head, sd.k_row,
                          sd.v_batch, sd.v_head, sd.v_row, sd.o_batch, sd.o_head, sd.o_row};
    for (int i = 0; i < 12; ++i)
        if (all[i] < 0 || all[i] % 8 != 0)
            return fail(MI355_ERR_BAD_ARGUMENT, "%s: stride %d is %ld; strides must be non-negative multiples of 8 elements", fn, i,
                        all[i]);
    if (sd.o_row < D || (Hq > 1 && sd.o_head < D) || (B > 1 && sd.o_batch < D))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: rows of O overlap (o strides %ld, %ld, %ld)", fn, sd.o_batch, sd.o_head, sd.o_row);
    if (ws.kind == mi355::FmhaWorkspace::kCaller) {
        const size_t need = mi355::fmha_decode_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len);
        if (need > 0 && (ws.ptr == nullptr || ws.bytes < need || reinterpret_cast<uintptr_t>(ws.ptr) % 16 != 0))
            return fail(MI355_ERR_BAD_ARGUMENT, "%s: workspace of %zu bytes at %p; this call needs %zu bytes, 16-byte aligned "
                        "(mi355_fmha_fwd_workspace_bytes)", fn, ws.bytes, ws.ptr, need);
    }
    hipError_t e = mi355::fmha_fwd_dispatch(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale, causal != 0, kv_valid_len, sd, dtype,
                                            variant, ws, static_cast<hipStream_t>(stream));
    if (e == hipErrorNotSupported)
        return fail(MI355_ERR_UNSUPPORTED, "%s: row strides of K and V must be below 2^24 elements (got %ld, %ld)", fn, sd.k_row, sd.v_row);
    if (e == hipErrorStreamCaptureUnsupported)
        return fail(static_cast<int>(e), "%s: the split-KV workspace of this stream would have to be allocated or enlarged while "
                    "the stream is capturing; run the call once before capture, or use mi355_fmha_fwd_ws", fn);
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

static int hgemm_silu_mul_impl(const char* fn, int dtype, const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                         int layout, void* stream) {
    if (!A || !B || !C) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if (M < 1 || N < 1 || K < 1) return fail(MI355_ERR_BAD_ARGUMENT, "%s: M, N, K must be >= 1", fn);
    if (layout != MI355_GEMM_NN && layout != MI355_GEMM_NT)
        return fail(MI355_ERR_UNSUPPORTED, "%s: layout %d has no fused epilogue (NN and NT do)", fn, layout);
    const int64_t b_min = (layout == MI355_GEMM_NT) ? K : 2 * (int64_t)N;
    if (lda < K || ldb < b_min || ldc < N)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: leading dimension too small", fn);
    if (N > 0x3fffffff) return fail(MI355_ERR_BAD_ARGUMENT, "%s: N too large", fn);
    hipError_t e = mi355::hgemm_silu_mul_dispatch(A, B, C, M, 2 * N, K, lda, ldb, ldc, layout, dtype, static_cast<hipStream_t>(stream));
    if (e == hipErrorNotSupported)
        return fail(MI355_ERR_UNSUPPORTED,
                    "%s: needs M <= 16 with layout NT, or M > 64 (or M > 16 with enough columns to fill the machine), N a multiple of 32, K a multiple of 64 and 16-byte aligned operands; "
                    "run mi355_hgemm and mi355_silu_mul(interleave = 32) instead", fn);
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

int mi355_hgemm_silu_mul(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                         int layout, void* stream) {
    return hgemm_silu_mul_impl("mi355_hgemm_silu_mul", MI355_DTYPE_FP16, A, B, C, M, N, K, lda, ldb, ldc, layout, stream);
}

int mi355_gemm_silu_mul_bf16(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                         int layout, void* stream) {
    return hgemm_silu_mul_impl("mi355_gemm_silu_mul_bf16", MI355_DTYPE_BF16, A, B, C, M, N, K, lda, ldb, ldc, layout, stream);
}


int mi355_fmha_fwd(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                   int Sk, int D, float scale, int causal, int kv_valid_len, void* stream) {
    return fmha_checked("mi355_fmha_fwd", Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len,
                        contiguous_strides(Hq, Hkv, Sq, Sk, D), MI355_DTYPE_FP16, stream);
}

int mi355_fmha_fwd_strided(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                           int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, void* stream) {
    if (!strides) return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd_strided: null strides");
    return fmha_checked("mi355_fmha_fwd_strided", Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len,
                        strides_from(strides), MI355_DTYPE_FP16, stream);
}

int mi355_fmha_fwd_bf16(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                        int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, void* stream) {
    return fmha_checked("mi355_fmha_fwd_bf16", Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len,
                        strides ? strides_from(strides) : contiguous_strides(Hq, Hkv, Sq, Sk, D), MI355_DTYPE_BF16, stream);
}

size_t mi355_fmha_fwd_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    if (B < 1 || Hq < 1 || Hkv < 1 || Sq < 1 || Sk < 1 || Hq % Hkv != 0 || kv_valid_len < 1 || kv_valid_len > Sk) return 0;
    return mi355::fmha_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len);
}

int mi355_fmha_fwd_ws(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                      int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, int dtype,
                      void* workspace, size_t workspace_bytes, void* stream) {
    if (dtype != MI355_DTYPE_FP16 && dtype != MI355_DTYPE_BF16)
        return fail(MI355_ERR_BAD_ARGUMENT, "mi355_fmha_fwd_ws: unknown dtype %d", dtype);
    mi355::FmhaWorkspace ws;
    ws.kind = mi355::FmhaWorkspace::kCaller;
    ws.ptr = workspace;
    ws.bytes = workspace_bytes;
    return fmha_checked("mi355_fmha_fwd_ws", Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len,
                        strides ? strides_from(strides) : contiguous_strides(Hq, Hkv, Sq, Sk, D), dtype, stream, 0, ws);
}

int mi355_fmha_fwd_noalloc(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                           int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, void* stream) {
    const char* fn = "mi355_fmha_fwd_noalloc";
    if (B >= 1 && Hq >= 1 && Hkv >= 1 && Sq >= 1 && Sk >= 1 && Hq % Hkv == 0 && kv_valid_len >= 1 && kv_valid_len <= Sk) {
        const size_t need = mi355::fmha_decode_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len);
        if (need > mi355::fmha_decode_static_scratch_bytes())
            return fail(MI355_ERR_UNSUPPORTED, "%s: the split-KV partial results of this call take %zu bytes, the static scratch "
                        "holds %zu; use mi355_fmha_fwd_ws with a workspace of your own", fn, need,
                        mi355::fmha_decode_static_scratch_bytes());
    }
    mi355::FmhaWorkspace ws;
    ws.kind = mi355::FmhaWorkspace::kStatic;
    return fmha_checked(fn, Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len,
                        strides ? strides_from(strides) : contiguous_strides(Hq, Hkv, Sq, Sk, D), MI355_DTYPE_FP16, stream, 0, ws);
}

int mi355_internal_fmha_fwd_variant(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                                    int Sq, int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides,
                                    int dtype, int variant, void* stream) {
    return fmha_checked("mi355_internal_fmha_fwd_variant", Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len,
                        strides ? strides_from(strides) : contiguous_strides(Hq, Hkv, Sq, Sk, D), dtype, stream, variant);
}

int mi355_internal_hgemm_variant(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb,
                                 int64_t ldc, int layout, int dtype, int variant, void* stream) {
    return hgemm_impl("mi355_internal_hgemm_variant", dtype, A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, layout, stream, variant);
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

static int rmsnorm_impl(const char* fn, int dtype, const void* x, const void* residual, void* residual_out, const void* weight, void* out, int64_t rows,
                  int hidden, int64_t ldx, int64_t ldr, int64_t ldro, int64_t ldo, float eps, void* stream) {
    if (!x || !weight || !out) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if ((residual == nullptr) != (residual_out == nullptr))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: residual and residual_out must both be given or both be NULL", fn);
    if (rows < 1 || hidden < 8 || hidden % 8 != 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: rows >= 1 and hidden a positive multiple of 8 required (got %lld, %d)", fn,
                    (long long)rows, hidden);
    if (ldx < hidden || ldo < hidden || ldx % 8 || ldo % 8 ||
        (residual && (ldr < hidden || ldro < hidden || ldr % 8 || ldro % 8)))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: row strides must be multiples of 8 and >= hidden", fn);
    if (!aligned16(x) || !aligned16(weight) || !aligned16(out) || !aligned16(residual) || !aligned16(residual_out))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
    if (!(eps >= 0.f) || eps > 1.f) return fail(MI355_ERR_BAD_ARGUMENT, "%s: eps outside [0, 1] (got %g)", fn, (double)eps);
    hipError_t e = mi355::rmsnorm_dispatch(x, residual, residual_out, weight, out, rows, hidden, ldx, ldr, ldro, ldo, eps, dtype,
                                           static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

int mi355_rmsnorm(const void* x, const void* residual, void* residual_out, const void* weight, void* out, int64_t rows,
                  int hidden, int64_t ldx, int64_t ldr, int64_t ldro, int64_t ldo, float eps, void* stream) {
    return rmsnorm_impl("mi355_rmsnorm", MI355_DTYPE_FP16, x, residual, residual_out, weight, out, rows, hidden, ldx, ldr, ldro, ldo, eps, stream);
}

int mi355_rmsnorm_bf16(const void* x, const void* residual, void* residual_out, const void* weight, void* out, int64_t rows,
                  int hidden, int64_t ldx, int64_t ldr, int64_t ldro, int64_t ldo, float eps, void* stream) {
    return rmsnorm_impl("mi355_rmsnorm_bf16", MI355_DTYPE_BF16, x, residual, residual_out, weight, out, rows, hidden, ldx, ldr, ldro, ldo, eps, stream);
}


static int rope_impl(const char* fn, int dtype, const void* x, void* out, int B, int S, int heads, int copy_heads, int D, int64_t x_batch, int64_t x_row,
               int64_t out_batch, int64_t out_row, const float* cos_table, const float* sin_table, const int32_t* positions,
               int64_t pos_batch, int n_positions, void* stream) {
    if (!x || !out || !cos_table || !sin_table || !positions) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if (D != 128) return fail(MI355_ERR_UNSUPPORTED, "%s: head_dim must be 128 (got %d)", fn, D);
    if (B < 1 || S < 1 || heads < 0 || copy_heads < 0 || heads + copy_heads < 1 || n_positions < 1 || pos_batch < 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: B, S, heads + copy_heads, n_positions must be >= 1, pos_batch >= 0", fn);
    const int64_t width = (int64_t)(heads + copy_heads) * D;
    if (x_row < width || out_row < width || x_row % 8 || out_row % 8 || x_batch % 8 || out_batch % 8 || x_batch < 0 || out_batch < 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: strides must be multiples of 8, row strides >= (heads + copy_heads) * 128", fn);
    if (!aligned16(x) || !aligned16(out) || !aligned16(cos_table) || !aligned16(sin_table))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
    hipError_t e = mi355::rope_dispatch(x, out, B, S, 0, heads, copy_heads, x_batch, x_row, out_batch, out_row, D, cos_table, sin_table,
                                        positions, pos_batch, n_positions, dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

static int rope_qkv_impl(const char* fn, int dtype, void* qkv, void* kv_out, int B, int S, int q_heads, int kv_heads, int D,
                         int64_t x_batch, int64_t x_row, int64_t out_batch, int64_t out_row, int64_t out_head, const float* cos_table,
                         const float* sin_table, const int32_t* positions, int64_t pos_batch, int n_positions, void* stream) {
    if (!qkv || !kv_out || !cos_table || !sin_table || !positions) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if (D != 128) return fail(MI355_ERR_UNSUPPORTED, "%s: head_dim must be 128 (got %d)", fn, D);
    if (B < 1 || S < 1 || q_heads < 1 || kv_heads < 1 || n_positions < 1 || pos_batch < 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: B, S, q_heads, kv_heads, n_positions must be >= 1, pos_batch >= 0", fn);
    const int64_t in_width = ((int64_t)q_heads + 2 * (int64_t)kv_heads) * D;
    if (x_row < in_width || out_row < D || out_head < D || x_row % 8 || out_row % 8 || out_head % 8 || x_batch % 8 || out_batch % 8 ||
        x_batch < 0 || out_batch < 0)
        return fail(MI355_ERR_BAD_ARGUMENT,
                    "%s: strides must be multiples of 8, x_row >= (q_heads + 2 kv_heads) * 128, out_row >= 128, out_head >= 128", fn);
    // heads side by side in a token row (out_head == 128) need a row that holds them all; a head-major cache (out_head >= a
    // head's whole sequence) needs rows of 128
    if (out_head < (int64_t)S * out_row && out_row < 2 * (int64_t)kv_heads * out_head)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: out_row / out_head make the heads of a token overlap those of the next", fn);
    if (!aligned16(qkv) || !aligned16(kv_out) || !aligned16(cos_table) || !aligned16(sin_table))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
    hipError_t e = mi355::rope_dispatch(qkv, kv_out, B, S, q_heads, q_heads + kv_heads, kv_heads, x_batch, x_row, out_batch, out_row,
                                        out_head, cos_table, sin_table, positions, pos_batch, n_positions, dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

int mi355_rope_qkv(void* qkv, void* kv_out, int B, int S, int q_heads, int kv_heads, int D, int64_t x_batch, int64_t x_row,
                   int64_t out_batch, int64_t out_row, int64_t out_head, const float* cos_table, const float* sin_table, const int32_t* positions,
                   int64_t pos_batch, int n_positions, void* stream) {
    return rope_qkv_impl("mi355_rope_qkv", MI355_DTYPE_FP16, qkv, kv_out, B, S, q_heads, kv_heads, D, x_batch, x_row, out_batch, out_row, out_head, cos_table, sin_table, positions, pos_batch, n_positions, stream);
}

int mi355_rope_qkv_bf16(void* qkv, void* kv_out, int B, int S, int q_heads, int kv_heads, int D, int64_t x_batch, int64_t x_row,
                        int64_t out_batch, int64_t out_row, int64_t out_head, const float* cos_table, const float* sin_table, const int32_t* positions,
                        int64_t pos_batch, int n_positions, void* stream) {
    return rope_qkv_impl("mi355_rope_qkv_bf16", MI355_DTYPE_BF16, qkv, kv_out, B, S, q_heads, kv_heads, D, x_batch, x_row, out_batch, out_row, out_head, cos_table, sin_table, positions, pos_batch, n_positions, stream);
}

int mi355_rope(const void* x, void* out, int B, int S, int heads, int copy_heads, int D, int64_t x_batch, int64_t x_row,
               int64_t out_batch, int64_t out_row, const float* cos_table, const float* sin_table, const int32_t* positions,
               int64_t pos_batch, int n_positions, void* stream) {
    return rope_impl("mi355_rope", MI355_DTYPE_FP16, x, out, B, S, heads, copy_heads, D, x_batch, x_row, out_batch, out_row, cos_table, sin_table, positions, pos_batch, n_positions, stream);
}

int mi355_rope_bf16(const void* x, void* out, int B, int S, int heads, int copy_heads, int D, int64_t x_batch, int64_t x_row,
               int64_t out_batch, int64_t out_row, const float* cos_table, const float* sin_table, const int32_t* positions,
               int64_t pos_batch, int n_positions, void* stream) {
    return rope_impl("mi355_rope_bf16", MI355_DTYPE_BF16, x, out, B, S, heads, copy_heads, D, x_batch, x_row, out_batch, out_row, cos_table, sin_table, positions, pos_batch, n_positions, stream);
}


static int silu_mul_impl(const char* fn, int dtype, const void* gate_up, void* out, int64_t rows, int inter, int interleave, int64_t ld_in, int64_t ld_out,
                   void* stream) {
    if (!gate_up || !out) return fail(MI355_ERR_BAD_ARGUMENT, "%s: null pointer", fn);
    if (rows < 1 || inter < 8 || inter % 8 != 0)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: rows >= 1 and inter a positive multiple of 8 required", fn);
    if (interleave < 0 || interleave % 8 != 0 || (interleave > 0 && inter % interleave != 0))
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: interleave must be 0 or a multiple of 8 that divides inter (got %d)", fn,
                    interleave);
    if (ld_in < 2 * (int64_t)inter || ld_out < inter || ld_in % 8 || ld_out % 8)
        return fail(MI355_ERR_BAD_ARGUMENT, "%s: ld_in >= 2 * inter, ld_out >= inter, both multiples of 8 required", fn);
    if (!aligned16(gate_up) || !aligned16(out)) return fail(MI355_ERR_BAD_ARGUMENT, "%s: pointers must be 16-byte aligned", fn);
    hipError_t e = mi355::silu_mul_dispatch(gate_up, out, rows, inter, interleave, ld_in, ld_out, dtype, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, fn);
    return 0;
}

int mi355_silu_mul(const void* gate_up, void* out, int64_t rows, int inter, int interleave, int64_t ld_in, int64_t ld_out,
                   void* stream) {
    return silu_mul_impl("mi355_silu_mul", MI355_DTYPE_FP16, gate_up, out, rows, inter, interleave, ld_in, ld_out, stream);
}

int mi355_silu_mul_bf16(const void* gate_up, void* out, int64_t rows, int inter, int interleave, int64_t ld_in, int64_t ld_out,
                   void* stream) {
    return silu_mul_impl("mi355_silu_mul_bf16", MI355_DTYPE_BF16, gate_up, out, rows, inter, interleave, ld_in, ld_out, stream);
}


const char* mi355_last_error(void) { return g_err; }

int mi355_serving_version(void) { return MI355_SERVING_VERSION; }

}  // extern "C"
