// Memory-bound layer glue around the GEMM and attention kernels for gfx950 (MI355X): RMSNorm (optionally fused with
// the residual add), rotary position embedding, SiLU(gate) * up. fp16 in/out, fp32 arithmetic, one rounding.
//
// These are the operations the reference's in-model path runs as separate PyTorch elementwise kernels between its
// calls of fine_fmha (benchmarks/flashattn-cuda/modeling_llama.py): LlamaRMSNorm.forward (:95-100), rotate_half /
// apply_rotary_pos_emb (:164-195), LlamaMLP.forward's act_fn(gate) * up (:227) and the residual adds of
// LlamaDecoderLayer.forward (:776-781). Each kernel moves every byte once with 16-byte accesses.
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
// out = weight * h * rsqrt(mean(h^2) + eps). The second pass re-reads the row (it is still in L2).
template <bool ADD>
__global__ __launch_bounds__(glue::THREADS) void rmsnorm_kernel(const half_t* x, const half_t* residual, half_t* res_out,
                                                                const half_t* __restrict__ weight, half_t* out,
                                                                int hidden, long ldx, long ldr, long ldro, long ldo,
                                                                float eps) {
    __shared__ float scratch[4];
    const long row = blockIdx.x;
    const half_t* xr = x + row * ldx;
    const half_t* rr = ADD ? residual + row * ldr : nullptr;
    half_t* ro = ADD ? res_out + row * ldro : nullptr;
    half_t* orow = out + row * ldo;
    float ss = 0.f;
    for (int c = threadIdx.x * 8; c < hidden; c += glue::THREADS * 8) {
        half8 v = *(const half8*)(xr + c);
        if (ADD) {
            half8 r = *(const half8*)(rr + c);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = (half_t)((float)v[j] + (float)r[j]);
            *(half8*)(ro + c) = v;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += (float)v[j] * (float)v[j];
    }
    const float total = glue::block_sum(ss, scratch);
    const float inv = __builtin_amdgcn_rsqf(total / (float)hidden + eps);
    for (int c = threadIdx.x * 8; c < hidden; c += glue::THREADS * 8) {
        half8 v = ADD ? *(const half8*)(ro + c) : *(const half8*)(xr + c);
        half8 w = *(const half8*)(weight + c);
        half8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (half_t)((float)w[j] * ((float)v[j] * inv));
        *(half8*)(orow + c) = o;
    }
}

// Rotary embedding of `heads` consecutive 128-wide heads per token: for i < 64
//   out[i]      = x[i] * cos[i]      - x[i + 64] * sin[i]
//   out[i + 64] = x[i + 64] * cos[i] + x[i] * sin[i]
// (rotate_half convention, modeling_llama.py:164-168,193-194), cos/sin rows of 64 fp32 selected by the token's position.
// The `copy_heads` heads that follow are moved unrotated (the value heads on their way into a KV cache).
// A thread owns 8 values of the lower half and their 8 partners; 8 threads per head, 32 heads per workgroup.
__global__ __launch_bounds__(glue::THREADS) void rope_kernel(const half_t* x, half_t* out, int S,
                                                             int heads, int copy_heads, long x_batch, long x_row, long o_batch,
                                                             long o_row, const float* __restrict__ cos_t,
                                                             const float* __restrict__ sin_t, const int* __restrict__ positions,
                                                             long pos_batch, int n_pos) {
    const long token = blockIdx.x;
    const int head = blockIdx.y * 32 + (threadIdx.x >> 3);
    if (head >= heads + copy_heads) return;
    const int i0 = (threadIdx.x & 7) * 8;
    const long b = token / S, s = token - b * S;
    const half_t* xp = x + b * x_batch + s * x_row + (long)head * 128 + i0;
    half_t* op = out + b * o_batch + s * o_row + (long)head * 128 + i0;
    const half8 lo = *(const half8*)xp;
    const half8 hi = *(const half8*)(xp + 64);
    if (head >= heads) {
        *(half8*)op = lo;
        *(half8*)(op + 64) = hi;
        return;
    }
    int pos = positions[b * pos_batch + s];
    pos = min(max(pos, 0), n_pos - 1);
    const float* cp = cos_t + (long)pos * 64 + i0;
    const float* sp = sin_t + (long)pos * 64 + i0;
    const float4v c0 = *(const float4v*)cp, c1 = *(const float4v*)(cp + 4);
    const float4v s0 = *(const float4v*)sp, s1 = *(const float4v*)(sp + 4);
    half8 olo, ohi;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float c = j < 4 ? c0[j] : c1[j - 4];
        const float sn = j < 4 ? s0[j] : s1[j - 4];
        const float a = (float)lo[j], bb = (float)hi[j];
        olo[j] = (half_t)(a * c - bb * sn);
        ohi[j] = (half_t)(bb * c + a * sn);
    }
    *(half8*)op = olo;
    *(half8*)(op + 64) = ohi;
}

// out[r][j] = silu(gate[r][j]) * up[r][j]. block == 0: gate = in[r][0 .. inter), up = in[r][inter .. 2 inter);
// block > 0 (a multiple of 8): gate and up alternate in groups of `block` columns, gate[j] = in[r][(j / block) * 2 block + j % block]
// and up[j] `block` columns further (the layout the GEMM's gate/up epilogue consumes).
__global__ __launch_bounds__(glue::THREADS) void silu_mul_kernel(const half_t* __restrict__ in, half_t* __restrict__ out,
                                                                 int inter, int block, long ld_in, long ld_out) {
    const long row = blockIdx.y;
    const int c = (blockIdx.x * glue::THREADS + threadIdx.x) * 8;
    if (c >= inter) return;
    const long gcol = block ? (long)(c / block) * 2 * block + c % block : c;
    const long ucol = block ? gcol + block : (long)inter + c;
    const half8 g = *(const half8*)(in + row * ld_in + gcol);
    const half8 u = *(const half8*)(in + row * ld_in + ucol);
    half8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float gf = (float)g[j];
        const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-gf * 1.4426950408889634f));
        o[j] = (half_t)(gf * sig * (float)u[j]);
    }
    *(half8*)(out + row * ld_out + c) = o;
}

hipError_t rmsnorm_dispatch(const void* x, const void* residual, void* res_out, const void* weight, void* out, long rows,
                            int hidden, long ldx, long ldr, long ldro, long ldo, float eps, hipStream_t stream) {
    if (rows > 0x7fffffffL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)rows), block(glue::THREADS);
    if (residual != nullptr)
        rmsnorm_kernel<true><<<grid, block, 0, stream>>>((const half_t*)x, (const half_t*)residual, (half_t*)res_out,
                                                         (const half_t*)weight, (half_t*)out, hidden, ldx, ldr, ldro, ldo, eps);
    else
        rmsnorm_kernel<false><<<grid, block, 0, stream>>>((const half_t*)x, nullptr, nullptr, (const half_t*)weight, (half_t*)out,
                                                          hidden, ldx, 0, 0, ldo, eps);
    return hipGetLastError();
}

hipError_t rope_dispatch(const void* x, void* out, int B, int S, int heads, int copy_heads, long x_batch, long x_row,
                         long o_batch, long o_row, const float* cos_t, const float* sin_t, const int* positions, long pos_batch,
                         int n_pos, hipStream_t stream) {
    const long tokens = (long)B * S;
    const int groups = (heads + copy_heads + 31) / 32;
    if (tokens > 0x7fffffffL || groups > 65535) return hipErrorInvalidValue;
    rope_kernel<<<dim3((unsigned)tokens, (unsigned)groups), dim3(glue::THREADS), 0, stream>>>(
        (const half_t*)x, (half_t*)out, S, heads, copy_heads, x_batch, x_row, o_batch, o_row, cos_t, sin_t, positions, pos_batch,
        n_pos);
    return hipGetLastError();
}

hipError_t silu_mul_dispatch(const void* in, void* out, long rows, int inter, int block, long ld_in, long ld_out,
                             hipStream_t stream) {
    if (rows > 65535L * 32768L) return hipErrorInvalidValue;
    // grid.y is limited to 65535: fold rows beyond that into several launches
    const unsigned gx = (unsigned)((inter / 8 + glue::THREADS - 1) / glue::THREADS);
    for (long r0 = 0; r0 < rows; r0 += 65535) {
        const long n = rows - r0 < 65535 ? rows - r0 : 65535;
        silu_mul_kernel<<<dim3(gx, (unsigned)n), dim3(glue::THREADS), 0, stream>>>((const half_t*)in + r0 * ld_in,
                                                                                  (half_t*)out + r0 * ld_out, inter, block, ld_in, ld_out);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace mi355
