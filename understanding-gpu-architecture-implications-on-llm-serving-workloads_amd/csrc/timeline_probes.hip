// Yardstick kernels of the profiling twin (libmi355_serving_timeline.so, built with -DMI355_TIMELINE; the product library
// does not contain this file). They measure what the machine gives to code that does nothing but one thing, so that the
// figures of the real kernels can be held against something measured on the same box with the same data:
//   * stream_read_kernel      a kernel that only reads: the ceiling of the bandwidth-bound kernels;
//   * mfma_only_kernel        matrix instructions back to back on register operands (N(0,1) or zeros), two waves per SIMD:
//                             what the matrix pipes sustain under the board's power limit;
//   * mfma_valu_kernel        on every SIMD one wave issues the matrix instructions of an attention key tile from registers
//                             while the other runs the softmax's instruction mix: how much of the VALU work the hardware
//                             really overlaps with matrix work of another wave (the ceiling of the ping-pong schedule).
// `bench.py --timeline --kernel-config stream_read_* | mfma_only_* | mfma_valu_*` launches them.
#include "mi355_common.h"
#include "mi355_timeline.h"

#ifdef MI355_TIMELINE
namespace mi355 {

__global__ __launch_bounds__(256) void stream_read_kernel(const float4v* __restrict__ p, long n16, float* sink) {
    float4v acc = {0.f, 0.f, 0.f, 0.f};
    const long stride = (long)gridDim.x * blockDim.x;
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        float4v v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; i < n16; i += stride) acc += p[i];
    if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) sink[0] = 1.f;   // keeps the loads alive; never true for the bench's data
}

// Operand registers are filled from `fill` (8192 halfs: N(0,1) or zeros, chosen by the caller); SHAPE 16: 16x16x32, 32: 32x32x16.
// 32 independent-enough instructions per iteration (8 accumulators), nothing else in the loop.
template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_only_kernel(const half_t* __restrict__ fill, float* __restrict__ out, int iters) {
    const int tid = threadIdx.x;
    half8 a[4], b[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = *(const half8*)(fill + ((tid * 4 + i) % 1024) * 8);
#pragma unroll
    for (int i = 0; i < 2; ++i) b[i] = *(const half8*)(fill + ((tid * 2 + i + 977) % 1024) * 8);
    float sum = 0.f;
    if constexpr (SHAPE == 32) {
        float16v acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int m = 0; m < 32; ++m) acc[m % 8] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(m % 8) / 2], b[m % 2], acc[m % 8], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum += acc[i][e];
    } else {
        float4v acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = float4v{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int m = 0; m < 32; ++m) acc[m % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(m % 8) / 2], b[m % 2], acc[m % 8], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) sum += acc[i][e];
    }
    out[(long)blockIdx.x * blockDim.x + tid] = sum;
}

// Per workgroup: [cycles of wave 0 (matrix group), cycles of wave 4 (VALU group)] for `iters` rounds; a round of the matrix
// group is the 68 MFMA 16x16x32 (or 34 MFMA 32x32x16) of one attention key tile of a 32-query wave, a round of the VALU group
// the softmax of such a tile (16 v_max3, 32 v_fma, 32 v_exp, 16 v_cvt_pk). mode bit 0: waves 0..3 run, bit 1: waves 4..7 run,
// bit 2 (16x16x32 only): the matrix wave reads its A operands from LDS as the attention kernel does (32 fragments per tile).
// No barriers and no memory traffic inside the rounds: the only thing the two waves of a SIMD share is the SIMD.
static __device__ unsigned long long mfma_valu_cycles[256 * 2];

template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_valu_kernel(const half_t* __restrict__ fill, float* __restrict__ out, int iters, int mode) {
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    __shared__ __attribute__((aligned(1024))) char lds_raw[65536];
    MI355_LDS char* lds = (MI355_LDS char*)lds_raw;
    for (int i = tid; i < 65536 / 2; i += 512) ((MI355_LDS half_t*)lds)[i] = fill[i % 8192];
    __syncthreads();
    float sum = 0.f;
    unsigned long long t0 = 0, t1 = 0;
    if (wave < 4) {
        if (mode & 1) {
            half8 a[4], b[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = *(const half8*)(fill + ((tid * 4 + i) % 1024) * 8);
#pragma unroll
            for (int i = 0; i < 2; ++i) b[i] = *(const half8*)(fill + ((tid * 2 + i + 977) % 1024) * 8);
            __builtin_amdgcn_s_setprio(1);
            if constexpr (SHAPE == 32) {
                float16v acc[6];
#pragma unroll
                for (int i = 0; i < 6; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
                t0 = timeline::shader_cycles();
                for (int it = 0; it < iters; ++it) {
#pragma unroll
                    for (int m = 0; m < 34; ++m) acc[m % 6] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m % 4], b[m % 2], acc[m % 6], 0, 0, 0);
                }
                t1 = timeline::shader_cycles();
#pragma unroll
                for (int i = 0; i < 6; ++i)
#pragma unroll
                    for (int e = 0; e < 16; ++e) sum += acc[i][e];
            } else {
                float4v acc[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = float4v{0.f, 0.f, 0.f, 0.f};
                if (mode & 4) {
                    // as the attention kernel's matrix phase: every pair of MFMAs takes its A operand from a fragment read
                    // from LDS six fragments earlier (16 ds_read_b128, then 16 pairs of ds_read_b64_tr_b16 per tile)
                    const int lane = tid & 63;
                    MI355_LDS char* base = lds + (wave & 3) * 16384;
                    const int koff = (lane & 15) * 256 + (((lane >> 4) ^ (lane & 15)) << 4);
                    const int vrow = 4 * (lane >> 4) + ((lane & 15) >> 2);
                    const int voff = vrow * 256 + (((((lane & 15) & 3) >> 1) ^ ((vrow & 7) << 1)) << 4) + (lane & 1) * 8;
                    auto rd = [&](int f) -> half8 {
                        if (f < 16) return lds_read_b128(base + ((koff ^ ((f >> 2) << 6)) + (f & 3) * 4096));
                        const int off = (voff ^ (((f - 16) & 7) << 5)) + (32 * ((f - 16) >> 3)) * 256;
                        return concat(lds_read_tr16_b64(base + off), lds_read_tr16_b64(base + off + 4096));
                    };
                    half8 fr[6];
                    t0 = timeline::shader_cycles();
                    for (int it = 0; it < iters; ++it) {
#pragma unroll
                        for (int i = 0; i < 6; ++i) fr[i] = rd(i);
#pragma unroll
                        for (int f = 0; f < 32; ++f) {
                            __builtin_amdgcn_sched_barrier(0);
                            acc[(2 * f) % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fr[f % 6], b[0], acc[(2 * f) % 8], 0, 0, 0);
                            acc[(2 * f + 1) % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fr[f % 6], b[1], acc[(2 * f + 1) % 8], 0, 0, 0);
                            if (f % 8 == 3) {
                                acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[0], b[0], acc[0], 0, 0, 0);
                                if (f < 16) acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[0], b[1], acc[1], 0, 0, 0);
                            }
                            if (f + 6 < 32) fr[f % 6] = rd(f + 6);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    t1 = timeline::shader_cycles();
                } else {
                t0 = timeline::shader_cycles();
                for (int it = 0; it < iters; ++it) {
#pragma unroll
                    for (int m = 0; m < 68; ++m) acc[m % 8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[m % 4], b[m % 2], acc[m % 8], 0, 0, 0);
                }
                t1 = timeline::shader_cycles();
                }
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e) sum += acc[i][e];
            }
        }
    } else if (mode & 2) {
        float s[32];
#pragma unroll
        for (int e = 0; e < 32; ++e) s[e] = (float)fill[(tid * 32 + e) % 8192];
        const float c = 0.1275f;
        float m_run = 1.0f;
        half8 pk[4];
        t0 = timeline::shader_cycles();
        for (int it = 0; it < iters; ++it) {
            float a = s[0], b2 = s[1];
#pragma unroll
            for (int e = 2; e < 32; e += 4) {
                asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(a) : "v"(a), "v"(s[e]), "v"(s[e + 1]));
                if (e + 3 < 32) asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(b2) : "v"(b2), "v"(s[e + 2]), "v"(s[e + 3]));
            }
            asm volatile("v_max3_f32 %0, %1, %2, %2" : "=v"(a) : "v"(a), "v"(b2), "v"(b2));
            m_run = a * 1e-30f;   // keeps the maximum alive without changing the data
            const float neg = -m_run * c;
            float x[32];
#pragma unroll
            for (int e = 0; e < 32; ++e) asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(x[e]) : "v"(s[e]), "v"(c), "v"(neg));
#pragma unroll
            for (int e = 0; e < 32; ++e) asm volatile("v_exp_f32 %0, %1" : "=v"(x[e]) : "v"(x[e]));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                int4v w;
#pragma unroll
                for (int e = 0; e < 4; ++e) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(w[e]) : "v"(x[8 * j + 2 * e]), "v"(x[8 * j + 2 * e + 1]));
                pk[j] = __builtin_bit_cast(half8, w);
            }
            asm volatile("" : "+v"(pk[0]), "+v"(pk[1]), "+v"(pk[2]), "+v"(pk[3]));
        }
        t1 = timeline::shader_cycles();
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) sum += (float)pk[j][e];
        sum += m_run;
    }
    if ((tid & 63) == 0 && (wave == 0 || wave == 4) && blockIdx.x < 256) mfma_valu_cycles[blockIdx.x * 2 + (wave >> 2)] = t1 - t0;
    out[(long)blockIdx.x * blockDim.x + tid] = sum;
}

}  // namespace mi355

extern "C" int mi355_timeline_stream_read(const void* src, size_t bytes, void* sink, void* stream) {
    if (src == nullptr || sink == nullptr || bytes % 16 != 0 || reinterpret_cast<uintptr_t>(src) % 16 != 0) return (int)hipErrorInvalidValue;
    mi355::stream_read_kernel<<<dim3(256), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const mi355::float4v*>(src), (long)(bytes / 16), static_cast<float*>(sink));
    return (int)hipGetLastError();
}

// fill: 8192 fp16 values on the device; out: 256 * 512 floats on the device. One workgroup of 8 waves per CU.
extern "C" int mi355_timeline_mfma_only(int shape, const void* fill, void* out, int iters, void* stream) {
    if (fill == nullptr || out == nullptr || iters < 1 || (shape != 16 && shape != 32)) return (int)hipErrorInvalidValue;
    auto st = static_cast<hipStream_t>(stream);
    if (shape == 32) mi355::mfma_only_kernel<32><<<dim3(256), dim3(512), 0, st>>>(static_cast<const mi355::half_t*>(fill), static_cast<float*>(out), iters);
    else mi355::mfma_only_kernel<16><<<dim3(256), dim3(512), 0, st>>>(static_cast<const mi355::half_t*>(fill), static_cast<float*>(out), iters);
    return (int)hipGetLastError();
}

extern "C" int mi355_timeline_mfma_valu(int shape, const void* fill, void* out, int iters, int mode, void* stream) {
    if (fill == nullptr || out == nullptr || iters < 1 || (shape != 16 && shape != 32) || mode < 1 || mode > 7) return (int)hipErrorInvalidValue;
    auto st = static_cast<hipStream_t>(stream);
    if (shape == 32) mi355::mfma_valu_kernel<32><<<dim3(256), dim3(512), 0, st>>>(static_cast<const mi355::half_t*>(fill), static_cast<float*>(out), iters, mode);
    else mi355::mfma_valu_kernel<16><<<dim3(256), dim3(512), 0, st>>>(static_cast<const mi355::half_t*>(fill), static_cast<float*>(out), iters, mode);
    return (int)hipGetLastError();
}

// [workgroup][0: matrix wave, 1: VALU wave] cycles of the last mfma_valu launch
extern "C" int mi355_timeline_read_mfma_valu(void* dst, size_t bytes) {
    const size_t all = sizeof(unsigned long long) * 256 * 2;
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(mi355::mfma_valu_cycles), bytes < all ? bytes : all);
}
#endif
