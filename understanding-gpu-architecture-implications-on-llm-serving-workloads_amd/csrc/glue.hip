// Memory-bound layer glue around the GEMM and attention kernels for gfx950 (MI355X): RMSNorm (optionally fused with
// the residual add), rotary position embedding, SiLU(gate) * up. fp16 in/out, fp32 arithmetic, one rounding.
//
// These are the operations the reference's in-model path runs as separate PyTorch elementwise kernels between its
// calls of fine_fmha (benchmarks/flashattn-cuda/modeling_llama.py): LlamaRMSNorm.forward (:95-100), rotate_half /
// apply_rotary_pos_emb (:164-195), LlamaMLP.forward's act_fn(gate) * up (:227) and the residual adds of
// LlamaDecoderLayer.forward (:776-781). Each kernel moves every byte once with 16-byte accesses.
#include <type_traits>

#include "mi355_common.h"
#include "mi355_serving_internal.h"

namespace mi355 {

namespace glue {

constexpr int THREADS = 256;

// sum over the 256 threads of a workgroup, result in every thread
__device__ __forceinline__ float block_sum(float x, float* scratch) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) scratch[wave] = x;
    __syncthreads();
    float t = scratch[0] + scratch[1] + scratch[2] + scratch[3];
    __syncthreads();
    return t;
}

}  // namespace glue

// One workgroup per row. ADD: h = residual + x is rounded to fp16, written to `res_out` (which may be `residual`
// itself), and normalised (the rounded value is what the next layer sees, so it is also what gets normalised).
// Otherwise h = x.
// out = weight * h * rsqrt(mean(h^2) + eps).
// REGS > 0: hidden <= REGS * 2048, the row and the weight stay in registers (REGS 16-byte pieces per thread each): every
// load of the kernel is issued up front, so a row costs one memory round trip, the sum and the store. On the 8 rows of a
// generation step the kernel is nothing but its chain of round trips (4.5 us with the weight fetched behind the sum and
// the row read a second time). REGS == 0: any hidden; the second pass re-reads the row (it is still in L2).
template <typename T, bool ADD, int REGS>
__global__ __launch_bounds__(glue::THREADS) void rmsnorm_kernel(const T* x, const T* residual, T* res_out,
                                                                const T* __restrict__ weight, T* out,
                                                                int hidden, long ldx, long ldr, long ldro, long ldo,
                                                                float eps) {
    using V8 = typename Elem<T>::v8;
    __shared__ float scratch[4];
    const long row = blockIdx.x;
    const T* xr = x + row * ldx;
    const T* rr = ADD ? residual + row * ldr : nullptr;
    T* ro = ADD ? res_out + row * ldro : nullptr;
    T* orow = out + row * ldo;
    float ss = 0.f;
    if constexpr (REGS > 0) {
        V8 v[REGS], r[REGS], w[REGS];
#pragma unroll
        for (int i = 0; i < REGS; ++i) {
            const int c = (i * glue::THREADS + threadIdx.x) * 8;
            if (c < hidden) {
                v[i] = *(const V8*)(xr + c);
                if (ADD) r[i] = *(const V8*)(rr + c);
                w[i] = *(const V8*)(weight + c);
            }
        }
#pragma unroll
        for (int i = 0; i < REGS; ++i) {
            const int c = (i * glue::THREADS + threadIdx.x) * 8;
            if (c < hidden) {
                if (ADD) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[i][j] = (T)((float)v[i][j] + (float)r[i][j]);
                    *(V8*)(ro + c) = v[i];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) ss += (float)v[i][j] * (float)v[i][j];
            }
        }
        const float total = glue::block_sum(ss, scratch);
        const float inv = __builtin_amdgcn_rsqf(total / (float)hidden + eps);
#pragma unroll
        for (int i = 0; i < REGS; ++i) {
            const int c = (i * glue::THREADS + threadIdx.x) * 8;
            if (c < hidden) {
                V8 o;
#pragma unroll
                for (int j = 0; j < 8; ++j) o[j] = (T)((float)w[i][j] * ((float)v[i][j] * inv));
                *(V8*)(orow + c) = o;
            }
        }
        return;
    }
    for (int c = threadIdx.x * 8; c < hidden; c += glue::THREADS * 8) {
        V8 v = *(const V8*)(xr + c);
        if (ADD) {
            V8 r = *(const V8*)(rr + c);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (T)((float)v[j] + (float)r[j]);
            *(V8*)(ro + c) = v;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += (float)v[j] * (float)v[j];
    }
    const float total = glue::block_sum(ss, scratch);
    const float inv = __builtin_amdgcn_rsqf(total / (float)hidden + eps);
    for (int c = threadIdx.x * 8; c < hidden; c += glue::THREADS * 8) {
        V8 v = ADD ? *(const V8*)(ro + c) : *(const V8*)(xr + c);
        V8 w = *(const V8*)(weight + c);
        V8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (T)((float)w[j] * ((float)v[j] * inv));
        *(V8*)(orow + c) = o;
    }
}

// Rotary embedding of `heads` consecutive 128-wide heads per token: for i < 64
//   out[i]      = x[i] * cos[i]      - x[i + 64] * sin[i]
//   out[i + 64] = x[i + 64] * cos[i] + x[i] * sin[i]
// (rotate_half convention, modeling_llama.py:164-168,193-194), cos/sin rows of 64 fp32 selected by the token's position.
// The `copy_heads` heads that follow are moved unrotated (the value heads on their way into a KV cache).
// The first `inplace_heads` heads are written back where they were read (the query heads of a fused QKV projection); the
// others go to `out`, whose head 0 is head `inplace_heads` of x (the key and value heads on their way into the cache),
// `o_head` elements from one head to the next (128 for heads side by side; a whole head's sequence for a head-major cache).
// A thread owns 8 values of the lower half and their 8 partners; 8 threads per head, 32 heads per workgroup.
template <typename T>
__global__ __launch_bounds__(glue::THREADS) void rope_kernel(const T* x, T* out, int S, int inplace_heads,
                                                             int heads, int copy_heads, long x_batch, long x_row, long o_batch,
                                                             long o_row, long o_head, const float* __restrict__ cos_t,
                                                             const float* __restrict__ sin_t, const int* __restrict__ positions,
                                                             long pos_batch, int n_pos) {
    using V8 = typename Elem<T>::v8;
    const long token = blockIdx.x;
    const int head = blockIdx.y * 32 + (threadIdx.x >> 3);
    if (head >= heads + copy_heads) return;
    const int i0 = (threadIdx.x & 7) * 8;
    const long b = token / S, s = token - b * S;
    const T* xp = x + b * x_batch + s * x_row + (long)head * 128 + i0;
    T* op = head < inplace_heads ? const_cast<T*>(xp) : out + b * o_batch + s * o_row + (long)(head - inplace_heads) * o_head + i0;
    const V8 lo = *(const V8*)xp;
    const V8 hi = *(const V8*)(xp + 64);
    if (head >= heads) {
        *(V8*)op = lo;
        *(V8*)(op + 64) = hi;
        return;
    }
    int pos = positions[b * pos_batch + s];
    pos = min(max(pos, 0), n_pos - 1);
    const float* cp = cos_t + (long)pos * 64 + i0;
    const float* sp = sin_t + (long)pos * 64 + i0;
    const float4v c0 = *(const float4v*)cp, c1 = *(const float4v*)(cp + 4);
    const float4v s0 = *(const float4v*)sp, s1 = *(const float4v*)(sp + 4);
    V8 olo, ohi;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float c = j < 4 ? c0[j] : c1[j - 4];
        const float sn = j < 4 ? s0[j] : s1[j - 4];
        const float a = (float)lo[j], bb = (float)hi[j];
        olo[j] = (T)(a * c - bb * sn);
        ohi[j] = (T)(bb * c + a * sn);
    }
    *(V8*)op = olo;
    *(V8*)(op + 64) = ohi;
}

// out[r][j] = silu(gate[r][j]) * up[r][j]. block == 0: gate = in[r][0 .. inter), up = in[r][inter .. 2 inter);
// block > 0 (a multiple of 8): gate and up alternate in groups of `block` columns, gate[j] = in[r][(j / block) * 2 block + j % block]
// and up[j] `block` columns further (the layout the GEMM's gate/up epilogue consumes).
template <typename T>
__global__ __launch_bounds__(glue::THREADS) void silu_mul_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                                 int inter, int block, long ld_in, long ld_out) {
    using V8 = typename Elem<T>::v8;
    const long row = blockIdx.y;
    const int c = (blockIdx.x * glue::THREADS + threadIdx.x) * 8;
    if (c >= inter) return;
    const long gcol = block ? (long)(c / block) * 2 * block + c % block : c;
    const long ucol = block ? gcol + block : (long)inter + c;
    const V8 g = *(const V8*)(in + row * ld_in + gcol);
    const V8 u = *(const V8*)(in + row * ld_in + ucol);
    V8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float gf = (float)g[j];
        const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-gf * 1.4426950408889634f));
        o[j] = (T)(gf * sig * (float)u[j]);
    }
    *(V8*)(out + row * ld_out + c) = o;
}

template <typename T>
static hipError_t rmsnorm_t(const void* x, const void* residual, void* res_out, const void* weight, void* out, long rows,
                            int hidden, long ldx, long ldr, long ldro, long ldo, float eps, hipStream_t stream) {
    if (rows > 0x7fffffffL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)rows), block(glue::THREADS);
    auto launch = [&](auto regs) {
        constexpr int REGS = decltype(regs)::value;
        if (residual != nullptr)
            rmsnorm_kernel<T, true, REGS><<<grid, block, 0, stream>>>((const T*)x, (const T*)residual, (T*)res_out, (const T*)weight,
                                                                      (T*)out, hidden, ldx, ldr, ldro, ldo, eps);
        else
            rmsnorm_kernel<T, false, REGS><<<grid, block, 0, stream>>>((const T*)x, nullptr, nullptr, (const T*)weight, (T*)out,
                                                                       hidden, ldx, 0, 0, ldo, eps);
    };
    if (hidden <= 2 * 2048) launch(std::integral_constant<int, 2>{});
    else if (hidden <= 4 * 2048) launch(std::integral_constant<int, 4>{});
    else launch(std::integral_constant<int, 0>{});
    return hipGetLastError();
}

hipError_t rmsnorm_dispatch(const void* x, const void* residual, void* res_out, const void* weight, void* out, long rows,
                            int hidden, long ldx, long ldr, long ldro, long ldo, float eps, int dtype, hipStream_t stream) {
    if (dtype == MI355_DTYPE_BF16) return rmsnorm_t<bf16_t>(x, residual, res_out, weight, out, rows, hidden, ldx, ldr, ldro, ldo, eps, stream);
    return rmsnorm_t<half_t>(x, residual, res_out, weight, out, rows, hidden, ldx, ldr, ldro, ldo, eps, stream);
}

hipError_t rope_dispatch(const void* x, void* out, int B, int S, int inplace_heads, int heads, int copy_heads, long x_batch,
                         long x_row, long o_batch, long o_row, long o_head, const float* cos_t, const float* sin_t, const int* positions, long pos_batch,
                         int n_pos, int dtype, hipStream_t stream) {
    const long tokens = (long)B * S;
    const int groups = (heads + copy_heads + 31) / 32;
    if (tokens > 0x7fffffffL || groups > 65535) return hipErrorInvalidValue;
    const dim3 grid((unsigned)tokens, (unsigned)groups), block(glue::THREADS);
    if (dtype == MI355_DTYPE_BF16)
        rope_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, S, inplace_heads, heads, copy_heads, x_batch, x_row,
                                                        o_batch, o_row, o_head, cos_t, sin_t, positions, pos_batch, n_pos);
    else
        rope_kernel<half_t><<<grid, block, 0, stream>>>((const half_t*)x, (half_t*)out, S, inplace_heads, heads, copy_heads, x_batch, x_row,
                                                        o_batch, o_row, o_head, cos_t, sin_t, positions, pos_batch, n_pos);
    return hipGetLastError();
}

hipError_t silu_mul_dispatch(const void* in, void* out, long rows, int inter, int block, long ld_in, long ld_out, int dtype,
                             hipStream_t stream) {
    if (rows > 65535L * 32768L) return hipErrorInvalidValue;
    // grid.y is limited to 65535: fold rows beyond that into several launches
    const unsigned gx = (unsigned)((inter / 8 + glue::THREADS - 1) / glue::THREADS);
    for (long r0 = 0; r0 < rows; r0 += 65535) {
        const long n = rows - r0 < 65535 ? rows - r0 : 65535;
        if (dtype == MI355_DTYPE_BF16)
            silu_mul_kernel<bf16_t><<<dim3(gx, (unsigned)n), dim3(glue::THREADS), 0, stream>>>(
                (const bf16_t*)in + r0 * ld_in, (bf16_t*)out + r0 * ld_out, inter, block, ld_in, ld_out);
        else
            silu_mul_kernel<half_t><<<dim3(gx, (unsigned)n), dim3(glue::THREADS), 0, stream>>>(
                (const half_t*)in + r0 * ld_in, (half_t*)out + r0 * ld_out, inter, block, ld_in, ld_out);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace mi355
