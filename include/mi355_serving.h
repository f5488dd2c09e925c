/*
 * mi355_serving.h -- C ABI of libmi355_serving.so: the fp16 GEMM and the fused multi-head-attention forward
 * for AMD Instinct MI355X (gfx950), as plain pointers and sizes. No torch types, no C++ types.
 *
 * This layer is what the PyTorch operators `gemm_unified::finegemm_N` and `fmha_unified::finefmha_N` call
 * after validating their tensors; it can equally be bound from C, C++ or ctypes.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; none is retained. The only memory the library ever
 *     allocates are three kinds of workspace. One holds the partial results of the split-KV attention path (taken when
 *     Hq/Hkv * Sq <= 32 and kv_valid_len >= 512, i.e. generation steps): one buffer per (device, stream), obtained
 *     with hipMalloc at first use (>= 4 MiB; when a later call needs more, a larger buffer is allocated and the old
 *     one is kept, because a HIP graph captured earlier may still hold its address; nothing is freed before the
 *     process ends, and every stream that ever made such a call keeps its buffer), so steady-state calls allocate
 *     nothing and calls on different streams never share a buffer.
 *     A call that would have to allocate while its stream is being captured fails (hipErrorStreamCaptureUnsupported)
 *     and launches nothing: run the step once on that stream before capturing it, and replay the graph on the stream it
 *     was captured on (or use mi355_fmha_fwd_ws with memory of your own). Only the calling stream's capture state is
 *     visible to the library: a first (or growing) call made while ANOTHER stream captures in global capture mode is a
 *     hipMalloc inside that capture and invalidates it, so make such calls before any capture starts.
 *     The GEMM entry points keep a second buffer of the same kind per (device, stream) for the partial tiles of their
 *     split-K path (17 .. 1024 rows against a second operand of up to 8192 columns, K a multiple of 128; >= 8 MiB, up to
 *     72 MiB); a GEMM call that cannot get it (its stream is being captured and has none yet, or hipMalloc fails) does not fail: it
 *     runs the kernels without split-K, so a captured call is faster when the step ran once on that stream before.
 *     The attention entry points other than mi355_fmha_fwd_ws (which takes the caller's) and mi355_fmha_fwd_noalloc
 *     (which walks all keys in one kernel) keep a third buffer of that kind
 *     for a chunk of queries against a long cache (at most 128 work items of 128 or 256 queries, kv_valid_len >= 2048: the keys
 *     are cut into up to 8 ranges and a second kernel merges the partial outputs, which take ranges * B * Hq * Sq * 260
 *     bytes; >= 8 MiB); a call that cannot get it walks all keys in one kernel instead of failing, like the GEMM;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); calls are asynchronous;
 *   - fp16 data is IEEE binary16 (`_Float16` / `__half` / torch.float16);
 *   - return value 0 = launched; non-zero = a hipError_t value or MI355_ERR_* below, nothing was launched.
 *     mi355_last_error() returns a thread-local description of the last failure.
 *   - calls are re-entrant and thread-safe, with one exception: mi355_fmha_fwd_noalloc, whose calls share one fixed
 *     array per GPU and must not overlap on a GPU (see there). The only other mutable global state is one-time kernel
 *     attribute initialisation (atomic flags) and the mutex-protected table of those workspaces. Which kernel runs
 *     depends on the arguments alone.
 */
#ifndef MI355_SERVING_H
#define MI355_SERVING_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_SERVING_VERSION 200

/* argument errors (distinct from hipError_t values, which are < 10000) */
#define MI355_ERR_BAD_ARGUMENT 10001
#define MI355_ERR_UNSUPPORTED 10002

/* element types (internal tags of the dispatchers; the entry points fix the type by name) */
#define MI355_DTYPE_FP16 0
#define MI355_DTYPE_BF16 1

/* operand layouts of mi355_hgemm */
#define MI355_GEMM_NN 0 /* A is [M,K] row-major, B is [K,N] row-major           */
#define MI355_GEMM_NT 1 /* A is [M,K] row-major, B is stored [N,K] (C = A * B^T) */
#define MI355_GEMM_TN 2 /* A is stored [K,M] (C = A^T * B), B is [K,N]           */

/*
 * C[M,N] (fp16, row-major, leading dimension ldc) = op(A) * op(B), fp32 accumulation, one rounding to fp16.
 *
 * Replaces the device side of the reference's host wrappers `at::Tensor finegemm_N(const at::Tensor& a,
 * const at::Tensor& b)`:
 *   layout NN  <- finegemm_0..11  (kernels/gemm/pkg/gemm_unified/csrc/auto/gemm_7.cu:111-151,
 *                                  semi/gemm_11_amd.cpp:129-154)
 *   layout TN  <- finegemm_12, 16 (manual/gemm_12_amd.cpp:294-316, manual/gemm_16_amd.cpp:345-367)
 *   layout NT  <- finegemm_13..15 (manual/gemm_13_amd.cpp:248-270, gemm_14_amd.cpp:268-290,
 *                                  gemm_15_amd.cpp:291-313)
 * lda/ldb/ldc are in elements and refer to the stored matrices (e.g. lda >= M for layout TN).
 * Any M, N, K >= 1 is accepted. The fast paths need A and B 16-byte aligned with lda and ldb multiples of 8, and
 * K % 8 == 0 (K % 64 != 0 with M <= 64 and no residual: one more launch for the last K % 64 columns); M and N are free
 * (ragged tile edges are handled inside the kernels; an operand whose M or N index is contiguous is read in 16-byte
 * chunks, up to 7 elements into the padding that its leading dimension, a multiple of 8, leaves behind M or N). C (and
 * a residual) may have any row stride and alignment (global memory takes 16-byte accesses at any element; only the
 * last N % 8 columns of a row are stored element by element).
 */
int mi355_hgemm(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb,
                int64_t ldc, int layout, void* stream);

/*
 * C[M,N] = silu(G) * U, where [G | U] = op(A) * op(B) and op(B) has 2N columns that alternate between 32 columns of G and
 * the matching 32 columns of U (column 64 b + c is G[:, 32 b + c] for c < 32 and U[:, 32 b + c - 32] for c >= 32): the
 * gate and up projections of a Llama MLP computed by one GEMM on an interleaved weight matrix, with the activation
 * applied to the accumulators before the single rounding to fp16. Replaces `self.act_fn(self.gate_proj(x)) * self.up_proj(x)`
 * (benchmarks/flashattn-cuda/modeling_llama.py:227): two GEMMs, a SiLU kernel and a multiply kernel in the reference.
 * Layouts NN and NT; N a multiple of 32, K a multiple of 64, 16-byte aligned operands and leading dimensions. Every such
 * shape is one launch: up to 16 rows in layout NT on the split-K small-M kernel, up to 64 rows otherwise on 64x64 tiles
 * with a deep ring (both stream the weight once), more rows on the 128x128 / 256x256 tiles, all with the same epilogue.
 * Other shapes (K or N off those multiples, unaligned operands, layout TN) return MI355_ERR_UNSUPPORTED and nothing is
 * launched: run mi355_hgemm on the same operands followed by mi355_silu_mul with interleave = 32.
 */
int mi355_hgemm_silu_mul(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                         int layout, void* stream);

/*
 * C[M,N] = R[M,N] + op(A) * op(B): the product of mi355_hgemm with a residual added in its epilogue, for the two
 * projections of a decoder layer whose result is added to the residual stream (`hidden_states = residual + hidden_states`
 * after o_proj and after down_proj, benchmarks/flashattn-cuda/modeling_llama.py:776,781; an elementwise kernel of its own
 * in the reference). The product is rounded to fp16 first and the sum once more, so the result equals that of the two
 * separate operations bit for bit (one exception: with K % 64 != 0 and M <= 64, mi355_hgemm forms its product in two
 * passes and this entry point in one, so the two may differ in the last bit of the product). R may be C (in place; then ldr must equal ldc), otherwise R and C must not overlap;
 * ldr >= N. Layouts, shapes and fast-path conditions as mi355_hgemm (R and ldr aligned like C and ldc).
 */
int mi355_hgemm_add(const void* A, const void* B, const void* R, void* C, int M, int N, int K, int64_t lda, int64_t ldb,
                    int64_t ldr, int64_t ldc, int layout, void* stream);

/*
 * Fused attention forward, O = softmax(scale * Q K^T + mask) V, online softmax with fp32 statistics.
 *
 * Replaces the device side of `torch::Tensor finefmha_N(Q, K, V, causal, is_decode, decode_length)`
 * (kernels/fmha/pkg/fmha_unified/csrc/semi/fmha_2_amd.cpp:311-359, auto/fmha_0.cu:301-330).
 *
 *   Q, O : [B, Hq,  Sq, D] fp16 contiguous ("BHSD")          K, V : [B, Hkv, Sk, D] fp16 contiguous
 *   LSE  : [B, Hq, Sq] fp32, natural-log log-sum-exp of the scaled, masked scores; may be NULL
 *   Hq % Hkv == 0; query head h reads kv head h / (Hq / Hkv)   (fmha_2_amd.cpp:33-42)
 *   D must be 128                                               (fmha_2_amd.cpp:329)
 *   kv_valid_len : keys with index >= kv_valid_len are masked (1 <= kv_valid_len <= Sk); this is the
 *                  `decode_length` argument of the reference with its off-by-one (`>`,
 *                  fmha_2_amd.cpp:191) corrected. Pass Sk for "all keys valid".
 *   causal != 0  : key j is visible to query i iff j <= i + (Sk - Sq), i.e. the mask is aligned to the
 *                  bottom-right corner; with Sq == Sk this is the reference's `q_pos < k_pos => masked`
 *                  rule (fmha_2_amd.cpp:187-190).
 *   scale        : softmax scale, positive and finite (the operators pass 1/sqrt(D), fmha_2_amd.cpp:320).
 *   Sq and Sk are arbitrary (>= 1); ragged tails are masked inside the kernel, no padding is needed.
 *   A query row with no visible key yields O = 0 and LSE = -inf.
 */
int mi355_fmha_fwd(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                   int Sq, int Sk, int D, float scale, int causal, int kv_valid_len, void* stream);

/*
 * mi355_fmha_fwd for operands that are not contiguous [B, H, S, D] tensors: element [b][h][s][d] of each operand
 * lives at b*batch + h*head + s*row + d, with d contiguous. `strides` holds 12 element strides in the order
 *   q_batch, q_head, q_row,  k_batch, k_head, k_row,  v_batch, v_head, v_row,  o_batch, o_head, o_row
 * each a non-negative multiple of 8 (16 bytes), k_row and v_row below 2^24; rows of O must not overlap. LSE stays
 * [B, Hq, Sq] contiguous.
 *
 * Replaces the copies the reference makes before its kernel: its callers hand over transposed views of
 * [B, S, H, D] projections (benchmarks/flashattn-cuda/modeling_llama.py:658-660) which
 * kernels/fmha/pkg/fmha_unified/ops.py:23-25 turns into contiguous tensors, and transpose the output back
 * (modeling_llama.py:700). With strides, Q/K/V can be read straight out of a fused QKV projection
 * ([B, S, (Hq + 2 Hkv) * D]: row = (Hq + 2 Hkv) * D, head = D) or a KV cache, and O written as [B, S, Hq * D].
 */
int mi355_fmha_fwd_strided(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                           int Sq, int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides,
                           void* stream);

/*
 * The same attention forward for bfloat16 Q, K, V, O (fp32 scores, statistics and accumulation as above; P is rounded to
 * bfloat16 for the second product). `strides` as in mi355_fmha_fwd_strided, or NULL for contiguous [B, H, S, D] tensors.
 * For callers of the reference's bf16 operator index (`finefmha_5`: kernels/fmha/pkg/fmha_unified/csrc/manual/fmha_5_nv.cu:148-150,
 * driven with bf16 tensors by kernels/fmha/test/perf.py:106-108 and the bf16 cases of correct.py:69-72).
 */
int mi355_fmha_fwd_bf16(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                        int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, void* stream);

/*
 * Layer glue between the GEMMs and the attention of a Llama decoder layer: memory-bound, fp16 in/out, fp32 arithmetic,
 * one rounding. They replace the separate PyTorch elementwise kernels of the reference's in-model path
 * (benchmarks/flashattn-cuda/modeling_llama.py). All pointers 16-byte aligned, all strides in elements and multiples of 8.
 *
 * mi355_rmsnorm: out[r] = weight * h[r] * rsqrt(mean(h[r]^2) + eps) over `hidden` columns   (LlamaRMSNorm.forward,
 *   modeling_llama.py:95-100). residual == NULL (then residual_out == NULL too): h = x. Otherwise h = fp16(residual + x), also
 *   written to residual_out (the `hidden_states = residual + hidden_states` that precedes each norm,
 *   modeling_llama.py:776-779); residual_out may be residual itself, and out may alias x.
 */
int mi355_rmsnorm(const void* x, const void* residual, void* residual_out, const void* weight, void* out, int64_t rows,
                  int hidden, int64_t ldx, int64_t ldr, int64_t ldro, int64_t ldo, float eps, void* stream);

/*
 * mi355_rope: rotary position embedding of `heads` consecutive 128-wide heads of every token (rotate_half convention,
 *   modeling_llama.py:164-168,193-194): for i < 64, with c = cos_table[p][i], s = sin_table[p][i],
 *   p = positions[b*pos_batch + t] (pos_batch = S for a [B, S] table, 0 when all batch rows share one [S] table):
 *     out[i] = x[i] c - x[i+64] s,   out[i+64] = x[i+64] c + x[i] s.
 *   Token (b, t) lives at x + b*x_batch + t*x_row (+ head*128), likewise for out, so q and k can be rotated inside a fused
 *   QKV projection (out == x) or k written straight into a KV cache. The `copy_heads` heads that follow the rotated ones are
 *   copied unrotated (the value heads, when k and v go into one cache tensor with a single launch). cos_table / sin_table: [n_positions][64] fp32, the
 *   first half of what LlamaRotaryEmbedding.forward builds (modeling_llama.py:119-132); positions outside
 *   [0, n_positions) are clamped.
 */
int mi355_rope(const void* x, void* out, int B, int S, int heads, int copy_heads, int D, int64_t x_batch, int64_t x_row,
               int64_t out_batch, int64_t out_row, const float* cos_table, const float* sin_table, const int32_t* positions,
               int64_t pos_batch, int n_positions, void* stream);

/*
 * mi355_rope_qkv: the two mi355_rope calls of a decoder layer with a KV cache in one launch. Token (b, t) of the fused
 *   projection lies at qkv + b*x_batch + t*x_row as [q_heads | kv_heads key heads | kv_heads value heads] of 128; the query
 *   heads are rotated in place; rotated key head h goes to kv_out + b*out_batch + t*out_row + h*out_head and value head h
 *   kv_heads heads further on. out_head = 128, out_row >= 2*kv_heads*128: K and V of a token side by side in a token-major
 *   cache [B, S_max, 2 kv_heads, 128]; out_row = 128, out_head = S_max*128: a head-major cache [B, 2 kv_heads, S_max, 128], in
 *   which every (sequence, head) is one contiguous stream for the generation-step attention (3 us faster at batch 8 over 8192
 *   keys than reading 256-byte pieces 4 KiB apart). Same tables, positions and arithmetic as mi355_rope: with out_head = 128
 *   the results are bit-identical to
 *   mi355_rope(qkv, qkv, .., q_heads, 0, ..) followed by mi355_rope(qkv + q_heads*128, kv_out, .., kv_heads, kv_heads, ..).
 *   (`query_states, key_states = apply_rotary_pos_emb(..)` and `past_key_value.update(key_states, value_states, ..)`,
 *   modeling_llama.py:664-668.)
 */
int mi355_rope_qkv(void* qkv, void* kv_out, int B, int S, int q_heads, int kv_heads, int D, int64_t x_batch, int64_t x_row,
                   int64_t out_batch, int64_t out_row, int64_t out_head, const float* cos_table, const float* sin_table, const int32_t* positions,
                   int64_t pos_batch, int n_positions, void* stream);

/*
 * mi355_silu_mul: out[r][j] = silu(g[r][j]) * u[r][j] (`act_fn(gate_proj(x)) * up_proj(x)`, modeling_llama.py:227, for gate
 *   and up computed by one GEMM). interleave == 0: g = gate_up[r][0 .. inter), u = gate_up[r][inter .. 2 inter).
 *   interleave == b > 0 (a multiple of 8 dividing inter): g and u alternate in groups of b columns, the layout
 *   mi355_hgemm_silu_mul consumes (b = 32).
 */
int mi355_silu_mul(const void* gate_up, void* out, int64_t rows, int inter, int interleave, int64_t ld_in, int64_t ld_out,
                   void* stream);

/*
 * bfloat16 twins of the fp16 entry points above: identical arguments and semantics, bfloat16 operands and results, fp32
 * accumulation and arithmetic (MFMA bf16 instructions with the fp16 kernels' tiling). For models whose checkpoints are
 * bfloat16; the reference's own bf16 use is its attention operator `finefmha_5` (see mi355_fmha_fwd_bf16).
 */
int mi355_gemm_bf16(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc,
                    int layout, void* stream);
int mi355_gemm_add_bf16(const void* A, const void* B, const void* R, void* C, int M, int N, int K, int64_t lda, int64_t ldb,
                        int64_t ldr, int64_t ldc, int layout, void* stream);
int mi355_gemm_silu_mul_bf16(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda, int64_t ldb,
                             int64_t ldc, int layout, void* stream);
int mi355_rmsnorm_bf16(const void* x, const void* residual, void* residual_out, const void* weight, void* out, int64_t rows,
                       int hidden, int64_t ldx, int64_t ldr, int64_t ldro, int64_t ldo, float eps, void* stream);
int mi355_rope_bf16(const void* x, void* out, int B, int S, int heads, int copy_heads, int D, int64_t x_batch, int64_t x_row,
                    int64_t out_batch, int64_t out_row, const float* cos_table, const float* sin_table,
                    const int32_t* positions, int64_t pos_batch, int n_positions, void* stream);
int mi355_rope_qkv_bf16(void* qkv, void* kv_out, int B, int S, int q_heads, int kv_heads, int D, int64_t x_batch, int64_t x_row,
                        int64_t out_batch, int64_t out_row, int64_t out_head, const float* cos_table, const float* sin_table,
                        const int32_t* positions, int64_t pos_batch, int n_positions, void* stream);
int mi355_silu_mul_bf16(const void* gate_up, void* out, int64_t rows, int inter, int interleave, int64_t ld_in, int64_t ld_out,
                        void* stream);

/*
 * The attention forward with a workspace owned by the caller, for callers that manage all device memory themselves
 * (HIP graph capture, arena allocators). mi355_fmha_fwd_workspace_bytes returns how many bytes a call with these sizes
 * needs: on the split-KV path 64 KiB of ticket counters plus the size of its partial results (at most ~9 MiB; 0 when
 * B * Hkv is large enough for one key range per (batch, kv head)); for a chunk of queries against a long cache (see the
 * conventions above) ranges * B * Hq * Sq * 260 bytes, which the call uses if `workspace_bytes` covers them and otherwise
 * does without (it then walks all keys in one kernel; a split-KV call with too small a workspace fails); 0 for every
 * other shape (then `workspace` may be NULL). mi355_fmha_fwd_ws is mi355_fmha_fwd_strided (strides == NULL:
 * contiguous [B, H, S, D] operands) for dtype MI355_DTYPE_FP16 or MI355_DTYPE_BF16 that keeps those partial results in
 * `workspace` (16-byte aligned, at least that many bytes, contents irrelevant before and after the call: a small kernel
 * clears the part that must start at zero) and never allocates. Calls that share a workspace must be ordered on one stream. No counterpart in the reference, whose
 * generation step runs the prefill kernel (kernels/fmha/pkg/fmha_unified/ops.py:19-25).
 */
size_t mi355_fmha_fwd_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len);
int mi355_fmha_fwd_ws(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                      int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, int dtype,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * mi355_fmha_fwd_strided (strides == NULL: contiguous [B, H, S, D] operands) for callers that cannot allocate device
 * memory at all: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. It has no
 * counterpart in the reference. It calls no hipMalloc / hipFree or any other allocating routine: the partial results of
 * the split-KV path live in a fixed 4 MiB array in device memory that is part of the library's code object (one copy
 * per GPU the library runs on, held until the process ends; its first 64 KiB hold the ticket counters). A call whose partial results do not fit (more than about
 * 7800 = (4 MiB - 64 KiB) / 528 B (workgroup, query column) pairs; a call runs about 256 workgroups, so this means more than ~30 query
 * rows per kv head at small batch; a Llama generation step has 4) returns MI355_ERR_UNSUPPORTED and launches nothing. Every call on a GPU shares that GPU's array: calls through this entry point
 * that overlap on one GPU (different streams, or threads) race; order them on one stream. The array's ticket counters are
 * zero when the library is loaded and every completed call leaves them at zero; a call that does not complete (an aborted
 * kernel, overlapping calls) can leave one that is not, and later calls for that (batch, kv head) then write no output
 * and report no error until the process ends (mi355_fmha_fwd_ws zeroes its counters on every call and has no such
 * memory). Shapes outside the split-KV path (prefill) do not touch the array and behave exactly like
 * mi355_fmha_fwd_strided.
 */
int mi355_fmha_fwd_noalloc(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                           int Sk, int D, float scale, int causal, int kv_valid_len, const int64_t* strides, void* stream);

/* Thread-local text for the last non-zero return of this thread ("" if none). */
const char* mi355_last_error(void);

/* MI355_SERVING_VERSION of the loaded library. */
int mi355_serving_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355_SERVING_H */
