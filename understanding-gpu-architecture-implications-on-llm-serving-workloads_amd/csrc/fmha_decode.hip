// Decode-shaped attention forward for gfx950 (MI355X): few query rows per kv head, long key sequence.
//
// The reference runs its generation step (`is_decode`, one query row padded to 64 by ops.py:19-25) through the
// prefill kernel, one workgroup per (batch, q head) walking all keys (semi/fmha_2_amd.cpp:341-356); that leaves
// almost the whole GPU idle and is bound by one workgroup's memory rate. Here the step is a split-KV
// ("flash-decoding") pass, HBM-bound by the single read of K and V:
//
//   pass 1  fmha_decode_split_kernel: a work unit is one wave = (batch, kv head, key range). The query rows of all
//           q heads that share the kv head are packed side by side as the (up to 32) columns of the S^T = K Q^T
//           product, so K and V are read once per kv head, not once per q head. The wave streams its key range in
//           tiles of 32 keys through its own LDS pipeline (direct-to-LDS copies, no workgroup barriers), runs the
//           same register-resident online softmax as the prefill kernel and writes unnormalised partial results
//           (O~ [128], m, l per column, fp32) to a workspace.
//   pass 2  fmha_decode_merge_kernel: one workgroup per query row combines the partials of all key ranges,
//           O = sum_s 2^((m_s - m) c) O~_s / sum_s 2^((m_s - m) c) l_s, and writes O (fp16) and LSE.
//
// Mask semantics are those of the prefill kernel (keys >= kv_valid_len masked; causal: key j visible to query i
// iff j <= i + Sk - Sq).
#include <atomic>
#include <map>
#include <mutex>
#include <utility>

#include "mi355_common.h"
#include "mi355_serving_internal.h"

namespace mi355 {

namespace dec {
constexpr int D = 128;
constexpr int TK = 32;                       // keys per tile
constexpr int ROW_BYTES = D * 2;             // 256
constexpr int TILE_BYTES = TK * ROW_BYTES;   // 8 KiB
constexpr int STAGE_BYTES = 2 * TILE_BYTES;  // K + V
constexpr int NSTAGE = 3;
constexpr int WAVES = 3;                     // work units per workgroup
constexpr int WAVE_BYTES = NSTAGE * STAGE_BYTES;
constexpr int LDS_BYTES = WAVES * WAVE_BYTES;  // 144 KiB
constexpr float kLazyLog2 = 8.f;             // rescale only when a column maximum grows by more than 2^8
constexpr int COPIES = 2 * (TILE_BYTES / 1024);  // 16 copy instructions per stage
constexpr int PART_STRIDE = D + 4;           // floats per (unit, column): O~[128], m, l, 2 pad (keeps rows 16-byte aligned)

__device__ __forceinline__ int swz_k(int row) { return row & 15; }
__device__ __forceinline__ int swz_v(int row) {
    int r = row & 3;
    return (r << 1) | ((r & 1) << 3);
}
__device__ __forceinline__ float other_half(float x) {
    int idx = ((int)(threadIdx.x & 63) ^ 32) << 2;
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(idx, __builtin_bit_cast(int, x)));
}
}  // namespace dec

// units = B * Hkv * splits, unit u = (b * Hkv + hkv) * splits + s covers key tiles [s * tiles_per_split, ...)
template <typename T>
__global__ __launch_bounds__(dec::WAVES * 64) void fmha_decode_split_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V, float* __restrict__ part, int B,
    int Hq, int Hkv, int Sq, int Sk, float scale_log2, int causal, int kv_valid, int splits, int tiles_per_split, int units, long q_batch,
    long q_head, long q_rstride, long k_batch, long k_head, long k_rstride, long v_batch, long v_head, long v_rstride) {
    using namespace dec;
    using V8 = typename Elem<T>::v8;
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = blockIdx.x * WAVES + wave;
    if (unit >= units) return;  // no workgroup barrier is used anywhere in this kernel
    MI355_LDS char* wbase = (MI355_LDS char*)smem_raw + wave * WAVE_BYTES;

    const int h = lane >> 5;
    const int l32 = lane & 31;
    const int s_idx = unit % splits;
    const int bh = unit / splits;
    const int hkv = bh % Hkv;
    const int b = bh / Hkv;
    const int group = Hq / Hkv;
    const int ncols = group * Sq;  // <= 32
    const int shift = Sk - Sq;

    // column c of the packed query block = (q head hkv*group + c / Sq, query row c % Sq)
    const int col = min(l32, ncols - 1);
    const int hq = hkv * group + col / Sq;
    const int qi = col % Sq;
    const T* qp = Q + b * q_batch + hq * q_head + qi * q_rstride + 8 * h;
    V8 qf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *(const V8*)(qp + ks * 16);
    const int lim = causal ? min(kv_valid - 1, qi + shift) : kv_valid - 1;  // last visible key of this column
    // smallest such limit over the wave: tiles that end at or before it need no mask code
    int lim_min = lim;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) lim_min = min(lim_min, __shfl_xor(lim_min, off, 64));
    lim_min = __builtin_amdgcn_readfirstlane(lim_min);

    const T* Kh = K + b * k_batch + hkv * k_head;
    const T* Vh = V + b * v_batch + hkv * v_head;

    const int tiles = (kv_valid + TK - 1) / TK;
    const int t_begin = s_idx * tiles_per_split;
    const int t_end = min(t_begin + tiles_per_split, tiles);

    // copy i (0..7) of a tile covers rows 4i + lane/16, chunk position lane%16
    const int c_row = lane >> 4;
    // addresses = wave-uniform tile base (scalar registers) + 32-bit lane offset; rows past the last valid key are
    // clamped onto it (masked later, but V must not feed NaNs into 0 * V)
    const uint32_t k_row_bytes = (uint32_t)k_rstride * 2, v_row_bytes = (uint32_t)v_rstride * 2;
    const uint32_t kcol = (lane & 15), c_row4 = c_row;
    auto issue_stage = [&](int tile, int slot) {
        MI355_LDS char* st = wbase + slot * STAGE_BYTES;
        const int tile_u = __builtin_amdgcn_readfirstlane(tile);
        const char* kb = (const char*)Kh + (long)tile_u * TK * k_rstride * 2;
        const char* vb = (const char*)Vh + (long)tile_u * TK * v_rstride * 2;
        const int last = kv_valid - 1 - tile_u * TK;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int row = 4 * i + c_row4;
            copy16_global_to_lds(kb, (uint32_t)min(row, last) * k_row_bytes + ((kcol ^ swz_k(row)) << 4), st + i * 1024);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int row = 4 * i + c_row4;
            copy16_global_to_lds(vb, (uint32_t)min(row, last) * v_row_bytes + ((kcol ^ swz_v(row)) << 4),
                                 st + TILE_BYTES + i * 1024);
        }
    };

    const int k_base = l32 * ROW_BYTES + ((h ^ (lane & 15)) << 4);  // xor (ks << 5)
    const int v_row = 4 * h + ((lane & 15) >> 2);
    const int v_clow = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    const int v_base = TILE_BYTES + v_row * ROW_BYTES + ((v_clow ^ swz_v(v_row)) << 4) + (lane & 1) * 8;  // xor (db << 6)

    float16v o[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const int n_loc = t_end - t_begin;
    // each wave starts at a different tile of its range and wraps around (the online softmax does not care about the
    // order): waves whose ranges lie a large power of two apart then do not walk the same memory channels in step
    const int rot = n_loc > 0 ? (unit * 5) % n_loc : 0;
    auto tile_of = [&](int i) { int r = i + rot; return t_begin + (r >= n_loc ? r - n_loc : r); };
    int issued = t_begin;
#pragma unroll
    for (int i = 0; i < NSTAGE - 1; ++i)
        if (issued < t_end) {
            issue_stage(tile_of(issued - t_begin), i);
            ++issued;
        }
    int slot = 0, fill = NSTAGE - 1;
    for (int tt0 = t_begin; tt0 < t_end; ++tt0) {
        const int t = tile_of(tt0 - t_begin);
        if (issued < t_end) {
            issue_stage(tile_of(issued - t_begin), fill);
            ++issued;
            fill = (fill + 1 == NSTAGE) ? 0 : fill + 1;
            wait_vmcnt<COPIES*(NSTAGE - 1)>();  // everything but the newest NSTAGE-1 tiles has landed
        } else {
            wait_vmcnt<0>();
        }
        MI355_LDS char* st = wbase + slot * STAGE_BYTES;
        slot = (slot + 1 == NSTAGE) ? 0 : slot + 1;

        // S^T = K Q^T : lane holds keys 8p + 4h + q of column l32
        float16v s;
#pragma unroll
        for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            V8 kf = Elem<T>::frag(lds_read_b128(st + (k_base ^ (ks << 5))));
            s = Elem<T>::mfma32(kf, qf[ks], s);
        }
        const int key0 = t * TK;
        if (key0 + TK - 1 > lim_min) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int key = key0 + 8 * (e >> 2) + 4 * h + (e & 3);
                if (key > lim) s[e] = -INFINITY;
            }
        }
        float mx = s[0];
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s[e]);
        mx = fmaxf(mx, other_half(mx));
        // lazy rescaling as in the prefill kernel: m_run is the exponent reference of the running sums and only moves
        // (with O and l rescaled) when some column exceeds it by more than 2^kLazyLog2
        const bool raise = (mx - m_run) * scale_log2 > kLazyLog2;  // -inf - -inf = NaN compares false
        if (__builtin_amdgcn_ballot_w64(raise) != 0) {
            float m_new = fmaxf(m_run, mx);
            float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * scale_log2);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
        }
        const float neg_ms = (m_run == -INFINITY) ? 0.f : -m_run * scale_log2;
        float psum = 0.f;
        V8 pf[2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            V8 pk;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[8 * tt + j], scale_log2, neg_ms));
                psum += p;
                pk[j] = (T)p;
            }
            pf[tt] = pk;
        }
        l_run += psum;
        // O^T += V^T P^T
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                int off = (v_base ^ (db << 6)) + (16 * tt) * ROW_BYTES;
                V8 vf = Elem<T>::frag(concat(lds_read_tr16_b64(st + off), lds_read_tr16_b64(st + off + 8 * ROW_BYTES)));
                o[db] = Elem<T>::mfma32(vf, pf[tt], o[db]);
            }
        wait_lgkmcnt<0>();  // the reads of this slot are complete before a later copy refills it
    }

    // partial result of this unit: O~ (unnormalised), m (raw score units), l
    const float l_tot = l_run + other_half(l_run);
    if (l32 < ncols) {
        float* pp = part + ((long)unit * ncols + l32) * PART_STRIDE;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                float4v v;
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = o[db][4 * p + q];
                *(float4v*)(pp + db * 32 + 8 * p + 4 * h) = v;
            }
        if (h == 0) {
            pp[D] = m_run;
            pp[D + 1] = l_tot;
        }
    }
}

// one workgroup of 128 threads per query row (b, hq, qi). The statistics of the key ranges are combined with the
// ranges spread over the threads (so their loads are independent), then thread d merges element d of O.
constexpr int kMaxSplits = 512;

template <typename T>
__global__ __launch_bounds__(128) void fmha_decode_merge_kernel(const float* __restrict__ part, T* __restrict__ O,
                                                                float* __restrict__ LSE, int Hq, int Hkv, int Sq,
                                                                float scale_log2, int splits, long o_batch, long o_head,
                                                                long o_row) {
    using namespace dec;
    using V8 = typename Elem<T>::v8;
    __shared__ float w_sh[kMaxSplits];
    __shared__ float red[128];
    const int tid = threadIdx.x;
    const int row = blockIdx.x;  // (b * Hq + hq) * Sq + qi
    const int qi = row % Sq;
    const int hq = (row / Sq) % Hq;
    const int b = row / (Sq * Hq);
    const int group = Hq / Hkv;
    const int hkv = hq / group;
    const int ncols = group * Sq;
    const int col = (hq - hkv * group) * Sq + qi;
    const float* base = part + (((long)(b * Hkv + hkv) * splits) * ncols + col) * PART_STRIDE;
    const long unit_stride = (long)ncols * PART_STRIDE;

    // m = max over ranges
    float m_loc = -INFINITY;
    for (int s = tid; s < splits; s += 128) {
        float ms = base[s * unit_stride + D];
        w_sh[s] = ms;
        m_loc = fmaxf(m_loc, ms);
    }
    red[tid] = m_loc;
    __syncthreads();
    float m = -INFINITY;
#pragma unroll 8
    for (int t = 0; t < 128; ++t) m = fmaxf(m, red[t]);
    __syncthreads();
    // weights 2^((m_s - m) c) (0 for ranges without a visible key) and l = sum_s w_s l_s
    float l_loc = 0.f;
    for (int s = tid; s < splits; s += 128) {
        float w = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((w_sh[s] - m) * scale_log2);
        w_sh[s] = w;
        l_loc += w * base[s * unit_stride + D + 1];
    }
    red[tid] = l_loc;
    __syncthreads();
    float l = 0.f;
#pragma unroll 8
    for (int t = 0; t < 128; ++t) l += red[t];
    // O[d] = sum_s w_s O~_s[d] / l
    float acc = 0.f;
#pragma unroll 8
    for (int s = 0; s < splits; ++s) acc += w_sh[s] * base[s * unit_stride + tid];
    O[b * o_batch + hq * o_head + qi * o_row + tid] = (T)((l > 0.f) ? acc / l : 0.f);
    if (LSE != nullptr && tid == 0)
        LSE[row] = (l > 0.f) ? (m * scale_log2 + __builtin_log2f(l)) * 0.69314718055994531f : -INFINITY;
}

bool fmha_decode_applicable(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    const int group = Hq / Hkv;
    return (long)group * Sq <= 32 && kv_valid_len >= 512 && Sk >= kv_valid_len && B >= 1;
}

// How a call is cut into work units, and what its partial results occupy.
struct DecodePlan {
    int splits, tiles_per_split;
    long units;
    size_t bytes;
};
static DecodePlan decode_plan(int B, int Hq, int Hkv, int Sq, int kv_valid) {
    using namespace dec;
    const int ncols = (Hq / Hkv) * Sq;
    const int tiles = (kv_valid + TK - 1) / TK;
    // about three waves (one workgroup) per CU in flight, at least 4 key tiles (128 keys) per wave
    int splits = (256 * WAVES) / (B * Hkv);
    splits = splits < 1 ? 1 : splits;
    const int max_splits = (tiles + 3) / 4;
    if (splits > max_splits) splits = max_splits;
    if (splits > kMaxSplits) splits = kMaxSplits;
    DecodePlan p;
    p.tiles_per_split = (tiles + splits - 1) / splits;
    p.splits = (tiles + p.tiles_per_split - 1) / p.tiles_per_split;
    p.units = (long)B * Hkv * p.splits;
    p.bytes = (size_t)p.units * ncols * PART_STRIDE * sizeof(float);
    return p;
}

size_t fmha_decode_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    if (!fmha_decode_applicable(B, Hq, Hkv, Sq, Sk, kv_valid_len)) return 0;
    return decode_plan(B, Hq, Hkv, Sq, kv_valid_len).bytes;
}

// The library's own workspace: one buffer per (device, stream), allocated on first use and replaced by a larger one when
// a call needs more. A buffer that has been handed to a kernel is NEVER freed: a HIP graph captured earlier may hold
// its address, so replaced buffers stay allocated until the process ends (each replacement is at least 1.5x larger, so
// together they hold less than three times the largest request). Calls on one stream are ordered, so they can share a
// buffer; calls on different streams get different ones. Nothing can be allocated while the stream is capturing: such a
// call fails with hipErrorStreamCaptureUnsupported unless an earlier call on the same stream already made the buffer
// large enough (run the step once before capturing it, or hand in a workspace of your own).
static hipError_t decode_workspace(size_t bytes, hipStream_t stream, float** out) {
    struct Buf {
        void* ptr = nullptr;
        size_t size = 0;
    };
    static std::mutex mu;
    static std::map<std::pair<int, hipStream_t>, Buf> bufs;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(mu);
    Buf& b = bufs[std::make_pair(dev, stream)];
    if (b.size < bytes) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &cap);
        if (e != hipSuccess) return e;
        if (cap != hipStreamCaptureStatusNone) return hipErrorStreamCaptureUnsupported;
        const size_t want = bytes < (size_t(4) << 20) ? (size_t(4) << 20) : bytes + bytes / 2;
        void* fresh = nullptr;
        e = hipMalloc(&fresh, want);
        if (e != hipSuccess) return e;
        b.ptr = fresh;   // the previous buffer, if any, stays allocated (see above)
        b.size = want;
    }
    *out = static_cast<float*>(b.ptr);
    return hipSuccess;
}

// Static scratch for callers that must not allocate (mi355_fmha_fwd_noalloc): a fixed array in device memory, one copy
// per GPU the library is loaded on, held until the process ends. Host code never uses the symbol's name as an address:
// the device address is looked up once per device with hipGetSymbolAddress and kept.
constexpr size_t kStaticScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

size_t fmha_decode_static_scratch_bytes() { return kStaticScratchBytes; }

static hipError_t static_scratch_ptr(float** out) {
    constexpr int kMaxDevices = 64;
    static std::atomic<void*> ptrs[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    void* p = ptrs[dev].load(std::memory_order_acquire);
    if (p == nullptr) {   // threads may race here; every one of them gets the same address for this device
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (p == nullptr) return hipErrorInvalidSymbol;
        ptrs[dev].store(p, std::memory_order_release);
    }
    *out = static_cast<float*>(p);
    return hipSuccess;
}

template <typename T>
hipError_t fmha_decode_dispatch(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq,
                                int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd,
                                const FmhaWorkspace& ws, hipStream_t stream) {
    using namespace dec;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(fmha_decode_split_kernel<T>), LDS_BYTES); e != hipSuccess) return e;
    const DecodePlan plan = decode_plan(B, Hq, Hkv, Sq, kv_valid);
    const int splits = plan.splits, tiles_per_split = plan.tiles_per_split;
    const long units = plan.units;

    float* part = nullptr;
    hipError_t e = hipSuccess;
    switch (ws.kind) {
        case FmhaWorkspace::kCaller:
            if (ws.ptr == nullptr || ws.bytes < plan.bytes || reinterpret_cast<uintptr_t>(ws.ptr) % 16 != 0) return hipErrorInvalidValue;
            part = static_cast<float*>(ws.ptr);
            break;
        case FmhaWorkspace::kStatic:
            if (plan.bytes > kStaticScratchBytes) return hipErrorOutOfMemory;   // the entry point checks first and says why
            e = static_scratch_ptr(&part);
            break;
        default:
            e = decode_workspace(plan.bytes, stream, &part);
            break;
    }
    if (e != hipSuccess) return e;
    const float scale_log2 = scale * 1.4426950408889634f;
    const unsigned blocks = (unsigned)((units + WAVES - 1) / WAVES);
    fmha_decode_split_kernel<T><<<dim3(blocks), dim3(WAVES * 64), LDS_BYTES, stream>>>(
        Q, K, V, part, B, Hq, Hkv, Sq, Sk, scale_log2, causal, kv_valid, splits, tiles_per_split, (int)units, sd.q_batch,
        sd.q_head, sd.q_row, sd.k_batch, sd.k_head, sd.k_row, sd.v_batch, sd.v_head, sd.v_row);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    fmha_decode_merge_kernel<T><<<dim3((unsigned)((long)B * Hq * Sq)), dim3(128), 0, stream>>>(
        part, O, LSE, Hq, Hkv, Sq, scale_log2, splits, sd.o_batch, sd.o_head, sd.o_row);
    return hipGetLastError();
}

template hipError_t fmha_decode_dispatch<half_t>(const half_t*, const half_t*, const half_t*, half_t*, float*, int, int, int, int,
                                                  int, float, int, int, const FmhaStrides&, const FmhaWorkspace&, hipStream_t);
template hipError_t fmha_decode_dispatch<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, bf16_t*, float*, int, int, int, int,
                                                 int, float, int, int, const FmhaStrides&, const FmhaWorkspace&, hipStream_t);

}  // namespace mi355
