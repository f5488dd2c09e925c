// Fused multi-head attention forward for gfx950 (MI355X), head_dim 128, fp16 in/out, fp32 softmax statistics.
//
// Replaces the reference's attention ladder (kernels/fmha/pkg/fmha_unified/csrc/{auto,semi}/fmha_*.{cu,cpp});
// semantics follow semi/fmha_2_amd.cpp: BHSD layout (:33-45), kv head = q head / (Hq/Hkv), causal rule
// "masked iff q_pos < k_pos" (:187-190), keys at or beyond the valid length masked (:191, with the off-by-one
// of the reference corrected), scale 1/sqrt(d) supplied by the caller (:320).
//
// Shape of the computation (per wave, everything stays in registers between the two matrix products):
//   S^T = K * Q^T      MFMA 32x32x16, A operand = K fragment read from LDS (ds_read_b128),
//                      B operand = Q fragment held in registers for the whole kernel.
//                      A lane then owns ONE query column (q = lane % 32) and 16 of the 32 keys of the block,
//                      so the softmax statistics m, l and the rescale factor are per-lane scalars.
//   P^T                exp2((S - m) * scale*log2e) in fp32, rounded to fp16; the accumulator layout of S^T is
//                      already the B-operand layout of the second product, so P never leaves the registers.
//   O^T += V^T * P^T   A operand = V^T fragment, read from the row-major V tile in LDS with the transposing
//                      ds_read_b64_tr_b16.
// K and V tiles (64 keys x 128 d) are copied global -> LDS with 16-byte direct-to-LDS copies, double buffered,
// 16-byte chunks XOR-swizzled so that both the b128 reads (K) and the transposing reads (V) are conflict free.
#include "mi355_common.h"
#include "mi355_serving_internal.h"

namespace mi355 {

namespace fmha {

constexpr int D = 128;            // head dim
constexpr int BN = 64;            // keys per tile
constexpr int ROW_BYTES = D * 2;  // 256
constexpr int TILE_BYTES = BN * ROW_BYTES;  // 16 KiB
constexpr int STAGE_BYTES = 2 * TILE_BYTES; // K + V
constexpr int NSTAGE = 2;
constexpr float kLazyLog2 = 8.f;  // rescale only when a row maximum grows by more than 2^8

__device__ __forceinline__ int swz_k(int row) { return row & 15; }
__device__ __forceinline__ int swz_v(int row) {
    int r = row & 3;
    return (r << 1) | ((r & 1) << 3);  // 0, 10, 4, 14
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// value held by the lane 32 positions away (lane ^ 32)
__device__ __forceinline__ float other_half(float x) {
    int idx = ((int)(threadIdx.x & 63) ^ 32) << 2;
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(idx, __builtin_bit_cast(int, x)));
}
// max / sum over the two 32-lane halves of the wave; result valid in all 64 lanes
__device__ __forceinline__ float halves_max(float x) { return fmaxf(x, other_half(x)); }
__device__ __forceinline__ float halves_sum(float x) { return x + other_half(x); }

}  // namespace fmha

// Decode the linear workgroup id into (batch, q head, q tile). Workgroups with ids congruent mod 8 share an
// XCD (and its L2): give each XCD whole (batch, kv head) groups so K/V are fetched from HBM once per XCD,
// and inside a group hand out the q tiles with the most keys (causal) first.
__device__ __forceinline__ void fmha_decode_block(int bid, int q_tiles, int group, int Hkv, int B, int& b, int& hq,
                                                  int& q_tile) {
    const int per_group = group * q_tiles;
    const int total = per_group * Hkv * B;
    int v = bid;
    if (total % 8 == 0) v = (bid % 8) * (total / 8) + bid / 8;
    int g = v / per_group;
    int r = v - g * per_group;
    int qt = r / group;
    int hin = r - qt * group;
    q_tile = q_tiles - 1 - qt;
    b = g / Hkv;
    hq = (g - b * Hkv) * group + hin;
}

template <typename T, int NQ, int NWAVES>
__global__ __launch_bounds__(NWAVES * 64, (NQ == 1 ? 2 : 1)) void fmha_fwd_kernel(const T* __restrict__ Q, const T* __restrict__ K,
                                                               const T* __restrict__ V, T* __restrict__ O,
                                                               float* __restrict__ LSE, int B, int Hq, int Hkv, int Sq,
                                                               int Sk, float scale_log2, int causal, int kv_valid,
                                                               int q_tiles, FmhaStrides sd) {
    using namespace fmha;
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    constexpr int BM = NWAVES * NQ * 32;
    constexpr int COPIES = (BN * ROW_BYTES / 1024) / NWAVES;  // wave-instructions per tile per wave
    static_assert(COPIES >= 1, "too many waves for the tile");

    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5;
    const int l32 = lane & 31;

    int b, hq, q_tile;
    const int group = Hq / Hkv;
    fmha_decode_block(blockIdx.x, q_tiles, group, Hkv, B, b, hq, q_tile);
    const int hkv = hq / group;

    const int q_block0 = q_tile * BM;            // first query row of the workgroup
    const int q_wave0 = q_block0 + wave * NQ * 32;  // first query row of this wave
    const int shift = Sk - Sq;

    const T* Qh = Q + b * sd.q_batch + hq * sd.q_head;
    const T* Kh = K + b * sd.k_batch + hkv * sd.k_head;
    const T* Vh = V + b * sd.v_batch + hkv * sd.v_head;
    T* Oh = O + b * sd.o_batch + hq * sd.o_head;

    // ---- number of key tiles this workgroup has to visit ----------------------------------------------
    int k_end = kv_valid;
    if (causal) {
        int last_q = min(q_block0 + BM, Sq) - 1;
        k_end = min(k_end, last_q + shift + 1);
    }
    const int n_tiles = (k_end + BN - 1) / BN;  // may be <= 0: no visible key for the whole tile

    // ---- Q fragments: lane holds Q[q = l32][d = 16*ks + 8*h .. +7] ---------------------------------------
    V8 qf[NQ][8];
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
        int qrow = min(q_wave0 + qb * 32 + l32, Sq - 1);
        const T* qp = Qh + qrow * sd.q_row + 8 * h;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[qb][ks] = *(const V8*)(qp + ks * 16);
    }

    // ---- global -> LDS copy bookkeeping ----------------------------------------------------------------
    // copy i of this wave covers tile rows (i*NWAVES + wave)*4 + lane/16, 16-byte chunk position lane%16
    int copy_row[COPIES];
    int copy_kcol[COPIES], copy_vcol[COPIES];
#pragma unroll
    for (int i = 0; i < COPIES; ++i) {
        int row = (i * NWAVES + wave) * 4 + (lane >> 4);
        copy_row[i] = row;
        copy_kcol[i] = ((lane & 15) ^ swz_k(row)) * 8;
        copy_vcol[i] = ((lane & 15) ^ swz_v(row)) * 8;
    }
    auto issue_copies = [&](int tile, int stage) {
        MI355_LDS char* sk = smem + stage * STAGE_BYTES;
        MI355_LDS char* sv = sk + TILE_BYTES;
#pragma unroll
        for (int i = 0; i < COPIES; ++i) {
            int krow = min(tile * BN + copy_row[i], kv_valid - 1);
            copy16_global_to_lds(Kh + krow * sd.k_row + copy_kcol[i], sk + (i * NWAVES + wave) * 1024);
        }
#pragma unroll
        for (int i = 0; i < COPIES; ++i) {
            int krow = min(tile * BN + copy_row[i], kv_valid - 1);
            copy16_global_to_lds(Vh + krow * sd.v_row + copy_vcol[i], sv + (i * NWAVES + wave) * 1024);
        }
    };

    // ---- LDS fragment offsets ----------------------------------------------------------------------------
    // K fragment (key block kb, k-step ks): row kb*32 + l32, chunk (2ks + h) ^ (row & 15)
    const int k_base = l32 * ROW_BYTES + ((h ^ (lane & 15)) << 4);  // xor (ks << 5), + kb * 32 * ROW_BYTES
    // V^T fragment (d block db): rows 4h + (lane%16)/4 (+ kb*32 + 16t + 8u), chunk (4db + clow) ^ swz_v(row)
    const int v_row = 4 * h + ((lane & 15) >> 2);
    const int v_clow = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    const int v_base = TILE_BYTES + v_row * ROW_BYTES + ((v_clow ^ swz_v(v_row)) << 4) + (lane & 1) * 8;  // xor (db << 6)

    float16v o[NQ][4];
    float m_run[NQ], l_run[NQ];
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
        m_run[qb] = -INFINITY;
        l_run[qb] = 0.f;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[qb][db][e] = 0.f;
    }

    if (n_tiles > 0) issue_copies(0, 0);

    for (int t = 0; t < n_tiles; ++t) {
        wait_vmcnt<0>();
        __syncthreads();
        if (t + 1 < n_tiles) issue_copies(t + 1, (t + 1) & 1);
        MI355_LDS char* st = smem + (t & 1) * STAGE_BYTES;
        const int key0 = t * BN;

        // ---- S^T = K Q^T ---------------------------------------------------------------------------------
        float16v s[NQ][2];
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) s[qb][kb][e] = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                V8 kf = Elem<T>::frag(lds_read_b128(st + ((k_base ^ (ks << 5)) + kb * 32 * ROW_BYTES)));
#pragma unroll
                for (int qb = 0; qb < NQ; ++qb)
                    s[qb][kb] = Elem<T>::mfma32(kf, qf[qb][ks], s[qb][kb]);
            }

        // ---- mask (only tiles that touch the diagonal or the end of the valid keys) ----------------------
        const bool need_mask = (key0 + BN > kv_valid) || (causal && (key0 + BN - 1 > q_wave0 + shift));
        if (need_mask) {
#pragma unroll
            for (int qb = 0; qb < NQ; ++qb) {
                int qi = q_wave0 + qb * 32 + l32;
                int lim = causal ? min(kv_valid - 1, qi + shift) : kv_valid - 1;  // last visible key
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        int key = key0 + kb * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                        if (key > lim) s[qb][kb][e] = -INFINITY;
                    }
            }
        }

        // ---- online softmax with lazy rescaling --------------------------------------------------------------
        // m_run is the exponent reference of the running sums, not necessarily the running maximum: it is only
        // raised (and O, l rescaled) when some row of the wave exceeds it by more than 2^kLazyLog2, which after the
        // first tiles almost never happens; until then P = exp2((S - m_run) * c) is at most 2^kLazyLog2, exact in
        // fp16/fp32 terms, and the final O / l and LSE do not depend on the choice of reference.
        V8 pf[NQ][2][2];
#pragma unroll
        for (int qb = 0; qb < NQ; ++qb) {
            float mx = s[qb][0][0];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[qb][kb][e]);
            mx = halves_max(mx);
            const bool raise = (mx - m_run[qb]) * scale_log2 > kLazyLog2;  // -inf - -inf = NaN compares false
            if (__builtin_amdgcn_ballot_w64(raise) != 0) {
                float m_new = fmaxf(m_run[qb], mx);
                float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                float alpha = fast_exp2((m_run[qb] - m_use) * scale_log2);
                m_run[qb] = m_new;
                l_run[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < 4; ++db)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[qb][db][e] *= alpha;
            }
            const float neg_ms = (m_run[qb] == -INFINITY) ? 0.f : -m_run[qb] * scale_log2;
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    float p = fast_exp2(__builtin_fmaf(s[qb][kb][e], scale_log2, neg_ms));
                    s[qb][kb][e] = p;
                    psum += p;
                }
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    V8 pk;
#pragma unroll
                    for (int j = 0; j < 8; ++j) pk[j] = (T)s[qb][kb][8 * tt + j];
                    pf[qb][kb][tt] = pk;
                }
            }
            l_run[qb] += psum;
        }

        // ---- O^T += V^T P^T ----------------------------------------------------------------------------------
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int db = 0; db < 4; ++db) {
                    int off = (v_base ^ (db << 6)) + (kb * 32 + 16 * tt) * ROW_BYTES;
                    half4 lo = lds_read_tr16_b64(st + off);
                    half4 hi = lds_read_tr16_b64(st + off + 8 * ROW_BYTES);
                    V8 vf = Elem<T>::frag(concat(lo, hi));
#pragma unroll
                    for (int qb = 0; qb < NQ; ++qb)
                        o[qb][db] = Elem<T>::mfma32(vf, pf[qb][kb][tt], o[qb][db]);
                }
    }

    // ---- finalize: O / l, LSE ---------------------------------------------------------------------------------
#pragma unroll
    for (int qb = 0; qb < NQ; ++qb) {
        float l_tot = halves_sum(l_run[qb]);
        float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
        int qi = q_wave0 + qb * 32 + l32;
        if (qi < Sq) {
            T* orow = Oh + qi * sd.o_row + 4 * h;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    V4 v;
#pragma unroll
                    for (int q = 0; q < 4; ++q) v[q] = (T)(o[qb][db][4 * p + q] * inv);
                    *(V4*)(orow + db * 32 + 8 * p) = v;
                }
            if (LSE != nullptr && h == 0) {
                float lse = (l_tot > 0.f) ? (m_run[qb] * scale_log2 + __builtin_log2f(l_tot)) * 0.69314718055994531f
                                          : -INFINITY;
                LSE[((long)b * Hq + hq) * (long)Sq + qi] = lse;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------
// Ping-pong kernel: 8 waves x 32 queries per workgroup, two waves per SIMD that alternate roles.
// Same mathematics and LDS layouts as fmha_fwd_kernel. A wave alternates between
//     an M phase: 16 MFMAs of S(j+1) = K(j+1) Q^T and 16 MFMAs of O += V(j)^T P(j)   (matrix pipe + LDS reads)
//     a  V phase: softmax of S(j+1) -> P(j+1)                                          (VALU only)
// separated by workgroup barriers. Waves 4..7 run one phase behind waves 0..3, so on every SIMD one wave is in
// its M phase while the other is in its V phase: the matrix pipe and the VALU are busy at the same time without
// relying on the instruction scheduler to interleave them inside one wave. The phases of the workgroup are
// numbered P0, P1, ...; waves 0..3 run M in the even ones, waves 4..7 in the odd ones.
// K and V have separate double buffers: tile j lives in Kbuf[j&1] / Vbuf[j&1], is copied by all 8 waves at the
// start of an even phase (K(i+1) and V(i) at P(2i)) and has two phases to land (waited for at the end of P(2i+1)).
// ---------------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(512, 2) void fmha_fwd_pingpong_kernel(const T* __restrict__ Q, const T* __restrict__ K,
                                                                   const T* __restrict__ V, T* __restrict__ O,
                                                                   float* __restrict__ LSE, int B, int Hq, int Hkv, int Sq,
                                                                   int Sk, float scale_log2, int causal, int kv_valid,
                                                                   int q_tiles, FmhaStrides sd) {
    using namespace fmha;
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    constexpr int NWAVES = 8;
    constexpr int BM = NWAVES * 32;
    constexpr int COPIES = (BN * ROW_BYTES / 1024) / NWAVES;  // 2 wave-instructions per tile per wave

    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;
    MI355_LDS char* kbuf = smem;                   // 2 x TILE_BYTES
    MI355_LDS char* vbuf = smem + 2 * TILE_BYTES;  // 2 x TILE_BYTES

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int late = wave >> 2;  // 0: waves 0..3 (M in even phases), 1: waves 4..7 (one phase behind)
    const int h = lane >> 5;
    const int l32 = lane & 31;

    int b, hq, q_tile;
    const int group = Hq / Hkv;
    fmha_decode_block(blockIdx.x, q_tiles, group, Hkv, B, b, hq, q_tile);
    const int hkv = hq / group;
    const int q_block0 = q_tile * BM;
    const int q_wave0 = q_block0 + wave * 32;
    const int shift = Sk - Sq;

    const T* Qh = Q + b * sd.q_batch + hq * sd.q_head;
    const T* Kh = K + b * sd.k_batch + hkv * sd.k_head;
    const T* Vh = V + b * sd.v_batch + hkv * sd.v_head;
    T* Oh = O + b * sd.o_batch + hq * sd.o_head;

    int k_end = kv_valid;
    if (causal) k_end = min(k_end, min(q_block0 + BM, Sq) - 1 + shift + 1);
    const int n_tiles = (k_end + BN - 1) / BN;  // may be <= 0: no visible key for the whole workgroup

    V8 qf[8];
    {
        int qrow = min(q_wave0 + l32, Sq - 1);
        const T* qp = Qh + qrow * sd.q_row + 8 * h;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = *(const V8*)(qp + ks * 16);
    }

    // copy i of this wave covers tile rows (i*NWAVES + wave)*4 + lane/16, 16-byte chunk position lane%16.
    // Addresses = wave-uniform tile base (scalar registers) + 32-bit lane offset; rows past the last valid key are
    // clamped onto it (they are masked later, but V must not feed NaNs into 0 * V).
    int copy_row[COPIES];
    uint32_t copy_kcol[COPIES], copy_vcol[COPIES];
#pragma unroll
    for (int i = 0; i < COPIES; ++i) {
        int row = (i * NWAVES + wave) * 4 + (lane >> 4);
        copy_row[i] = row;
        copy_kcol[i] = ((lane & 15) ^ swz_k(row)) * 16;
        copy_vcol[i] = ((lane & 15) ^ swz_v(row)) * 16;
    }
    const uint32_t k_row_bytes = (uint32_t)sd.k_row * 2, v_row_bytes = (uint32_t)sd.v_row * 2;
    auto issue_k = [&](int tile) {
        const char* base = (const char*)Kh + (long)tile * BN * sd.k_row * 2;
        const int last = kv_valid - 1 - tile * BN;
#pragma unroll
        for (int i = 0; i < COPIES; ++i)
            copy16_global_to_lds(base, (uint32_t)min(copy_row[i], last) * k_row_bytes + copy_kcol[i],
                                 kbuf + (tile & 1) * TILE_BYTES + (i * NWAVES + wave) * 1024);
    };
    auto issue_v = [&](int tile) {
        const char* base = (const char*)Vh + (long)tile * BN * sd.v_row * 2;
        const int last = kv_valid - 1 - tile * BN;
#pragma unroll
        for (int i = 0; i < COPIES; ++i)
            copy16_global_to_lds(base, (uint32_t)min(copy_row[i], last) * v_row_bytes + copy_vcol[i],
                                 vbuf + (tile & 1) * TILE_BYTES + (i * NWAVES + wave) * 1024);
    };

    const int k_base = l32 * ROW_BYTES + ((h ^ (lane & 15)) << 4);  // xor (ks << 5), + kb * 32 * ROW_BYTES
    const int v_row = 4 * h + ((lane & 15) >> 2);
    const int v_clow = 2 * ((lane >> 4) & 1) + ((lane & 3) >> 1);
    const int v_base = v_row * ROW_BYTES + ((v_clow ^ swz_v(v_row)) << 4) + (lane & 1) * 8;  // xor (db << 6)

    float16v o[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // The compiler is free to move register-only work across s_barrier; these empty asm statements make a value
    // "used" at a program point, which keeps the softmax in the V phase and the MFMAs in the M phase.
    auto pin_s = [](float16v(&s)[2]) { asm volatile("" : "+v"(s[0]), "+v"(s[1])); };
    auto pin_p = [](V8(&pf)[2][2]) { asm volatile("" : "+v"(pf[0][0]), "+v"(pf[0][1]), "+v"(pf[1][0]), "+v"(pf[1][1])); };
    auto pin_o = [&]() { asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3])); };

    // ---- phase bookkeeping -------------------------------------------------------------------------------------
    int phase = 0;  // index of the workgroup phase this wave is in
    // ends the current phase and starts the next one
    auto next_phase = [&]() {
        if (phase & 1) wait_vmcnt<0>();  // copies issued at the start of the previous (even) phase have landed
        __syncthreads();
        ++phase;
        if (!(phase & 1)) {
            const int i = phase >> 1;
            if (i + 1 < n_tiles) issue_k(i + 1);
            if (i < n_tiles) issue_v(i);
        }
    };

    // ---- building blocks ----------------------------------------------------------------------------------------
    // LDS fragment reads, named so the M phase below can issue them long before their MFMA
    auto read_k = [&](MI355_LDS char* kst, int kb, int ks) {
        return Elem<T>::frag(lds_read_b128(kst + ((k_base ^ (ks << 5)) + kb * 32 * ROW_BYTES)));
    };
    auto read_v = [&](MI355_LDS char* vst, int step) {  // step = (kb*2 + tt)*4 + db, the order the MFMAs consume them
        const int db = step & 3, tt = (step >> 2) & 1, kb = step >> 3;
        const int off = (v_base ^ (db << 6)) + (kb * 32 + 16 * tt) * ROW_BYTES;
        return Elem<T>::frag(concat(lds_read_tr16_b64(vst + off), lds_read_tr16_b64(vst + off + 8 * ROW_BYTES)));
    };
    // The M phase in the exact order it should issue: every fragment is read 8 MFMAs (256 cycles) before the MFMA
    // that consumes it, into the register its predecessor has just released. sched_barrier pins that order.
    //   MFMAs  0.. 7: S block 0 (K fragments read up front)        reads issued: K fragments of block 1
    //   MFMAs  8..15: S block 1                                     reads issued: V fragments 0..7
    //   MFMAs 16..23: O += V^T P, fragments 0..7                    reads issued: V fragments 8..15
    //   MFMAs 24..31: O += V^T P, fragments 8..15
    auto qk_tile = [&](int tile, float16v(&s)[2]) {  // S(tile) alone (first M phase of a wave)
        MI355_LDS char* kst = kbuf + (tile & 1) * TILE_BYTES;
        V8 kf[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) kf[i] = read_k(kst, 0, i);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_barrier(0);
                s[kb] = Elem<T>::mfma32(kf[i], qf[i], s[kb]);
                if (kb == 0) kf[i] = read_k(kst, 1, i);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto pv_tile = [&](int tile, const V8(&pf)[2][2]) {  // O += V(tile)^T P alone (last M phase of a wave)
        MI355_LDS char* vst = vbuf + (tile & 1) * TILE_BYTES;
        V8 vf[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) vf[i] = read_v(vst, i);
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_barrier(0);
                const int step = half * 8 + i;
                o[step & 3] = Elem<T>::mfma32(vf[i], pf[step >> 3][(step >> 2) & 1], o[step & 3]);
                if (half == 0) vf[i] = read_v(vst, 8 + i);
            }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto m_phase = [&](int tile_k, float16v(&s)[2], int tile_v, const V8(&pf)[2][2]) {  // S(tile_k) and O += V(tile_v)^T P
        MI355_LDS char* kst = kbuf + (tile_k & 1) * TILE_BYTES;
        MI355_LDS char* vst = vbuf + (tile_v & 1) * TILE_BYTES;
        V8 fr[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) fr[i] = read_k(kst, 0, i);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_barrier(0);
                s[kb] = Elem<T>::mfma32(fr[i], qf[i], s[kb]);
                fr[i] = (kb == 0) ? read_k(kst, 1, i) : read_v(vst, i);
            }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                __builtin_amdgcn_sched_barrier(0);
                const int step = half * 8 + i;
                o[step & 3] = Elem<T>::mfma32(fr[i], pf[step >> 3][(step >> 2) & 1], o[step & 3]);
                if (half == 0) fr[i] = read_v(vst, 8 + i);
            }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto softmax_tile = [&](float16v(&s)[2], int tile, V8(&pf)[2][2]) {
        const int key0 = tile * BN;
        const bool need_mask = (key0 + BN > kv_valid) || (causal && (key0 + BN - 1 > q_wave0 + shift));
        if (need_mask) {
            int qi = q_wave0 + l32;
            int lim = causal ? min(kv_valid - 1, qi + shift) : kv_valid - 1;  // last visible key
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    int key = key0 + kb * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                    if (key > lim) s[kb][e] = -INFINITY;
                }
        }
        float mx = s[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[kb][e]);
        mx = halves_max(mx);
        const bool raise = (mx - m_run) * scale_log2 > kLazyLog2;  // lazy rescaling, see fmha_fwd_kernel
        if (__builtin_amdgcn_ballot_w64(raise) != 0) {
            float m_new = fmaxf(m_run, mx);
            float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            float alpha = fast_exp2((m_run - m_use) * scale_log2);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
        }
        const float neg_ms = (m_run == -INFINITY) ? 0.f : -m_run * scale_log2;
        // In this phase the wave is the only one of its SIMD issuing VALU work, so dependent instructions must be
        // kept apart: all 32 multiply-adds, then all 32 exponentials, then four independent partial sums.
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) s[kb][e] = __builtin_fmaf(s[kb][e], scale_log2, neg_ms);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) s[kb][e] = fast_exp2(s[kb][e]);
        __builtin_amdgcn_sched_barrier(0);
        float ps[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                V8 pk;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    ps[j & 3] += s[kb][8 * tt + j];
                    pk[j] = (T)s[kb][8 * tt + j];
                }
                pf[kb][tt] = pk;
            }
        l_run += (ps[0] + ps[1]) + (ps[2] + ps[3]);
    };

    if (n_tiles > 0) {
        // before P0: K(0) must be in LDS
        issue_k(0);
        wait_vmcnt<0>();
        __syncthreads();
        if (1 < n_tiles) issue_k(1);  // start of P0
        issue_v(0);
        if (late) next_phase();  // waves 4..7 idle during P0

        float16v s[2];
        V8 pf[2][2];
        __builtin_amdgcn_s_setprio(1);
        qk_tile(0, s);
        __builtin_amdgcn_s_setprio(0);
        pin_s(s);
        next_phase();
        for (int j = 0; j + 1 < n_tiles; ++j) {
            softmax_tile(s, j, pf);  // V phase
            pin_p(pf);
            next_phase();
            __builtin_amdgcn_s_setprio(1);
            m_phase(j + 1, s, j, pf);
            __builtin_amdgcn_s_setprio(0);
            pin_s(s);
            pin_o();
            next_phase();
        }
        softmax_tile(s, n_tiles - 1, pf);
        pin_p(pf);
        next_phase();
        pv_tile(n_tiles - 1, pf);
        next_phase();
        if (!late) next_phase();  // waves 0..3 idle while waves 4..7 finish
    }

    // ---- finalize: O / l, LSE ---------------------------------------------------------------------------------
    float l_tot = halves_sum(l_run);
    float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    int qi = q_wave0 + l32;
    if (qi < Sq) {
        T* orow = Oh + qi * sd.o_row + 4 * h;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                V4 v;
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = (T)(o[db][4 * p + q] * inv);
                *(V4*)(orow + db * 32 + 8 * p) = v;
            }
        if (LSE != nullptr && h == 0) {
            float lse = (l_tot > 0.f) ? (m_run * scale_log2 + __builtin_log2f(l_tot)) * 0.69314718055994531f : -INFINITY;
            LSE[((long)b * Hq + hq) * (long)Sq + qi] = lse;
        }
    }
}

template <typename T>
static hipError_t launch_fmha_pingpong(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq,
                                       int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd,
                                       hipStream_t stream) {
    constexpr int BM = 256;
    constexpr int LDS = 4 * fmha::TILE_BYTES;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(fmha_fwd_pingpong_kernel<T>), LDS); e != hipSuccess) return e;
    const int q_tiles = (Sq + BM - 1) / BM;
    const long blocks = (long)q_tiles * Hq * B;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    const float scale_log2 = scale * 1.4426950408889634f;
    fmha_fwd_pingpong_kernel<T><<<dim3((unsigned)blocks), dim3(512), LDS, stream>>>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale_log2,
                                                                                causal, kv_valid, q_tiles, sd);
    return hipGetLastError();
}

template <typename T, int NQ, int NWAVES>
static hipError_t launch_fmha(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq,
                              int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd,
                                       hipStream_t stream) {
    constexpr int BM = NWAVES * NQ * 32;
    constexpr int LDS = fmha::STAGE_BYTES * fmha::NSTAGE;
    auto kern = fmha_fwd_kernel<T, NQ, NWAVES>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), LDS); e != hipSuccess) return e;
    const int q_tiles = (Sq + BM - 1) / BM;
    const long blocks = (long)q_tiles * Hq * B;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    const float scale_log2 = scale * 1.4426950408889634f;
    kern<<<dim3((unsigned)blocks), dim3(NWAVES * 64), LDS, stream>>>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale_log2,
                                                                    causal, kv_valid, q_tiles, sd);
    return hipGetLastError();
}

template <typename T>
static hipError_t fmha_fwd_dispatch_t(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                                      int Sq, int Sk, float scale, int causal, int kv_valid_len, const FmhaStrides& sd,
                                      int variant, const FmhaWorkspace& ws, hipStream_t stream) {
    const T* q = static_cast<const T*>(Q);
    const T* k = static_cast<const T*>(K);
    const T* v = static_cast<const T*>(V);
    T* o = static_cast<T*>(O);
    // the split-KV and ping-pong kernels address a K/V tile with 32-bit byte offsets from its first row
    const bool rows_fit_32bit = sd.k_row < (1L << 24) && sd.v_row < (1L << 24);
    if ((variant == 0 || variant == 4) && rows_fit_32bit && fmha_decode_applicable(B, Hq, Hkv, Sq, Sk, kv_valid_len))
        return fmha_decode_dispatch<T>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, ws, stream);
    if (variant == 0 || variant == 4) {
        // 256-query ping-pong workgroups once there are enough of them to fill the 256 CUs, otherwise 128-query ones
        const long wg256 = (long)((Sq + 255) / 256) * Hq * B;
        variant = (wg256 >= 256) ? 3 : 1;
    }
    if (variant == 3 && !rows_fit_32bit) variant = 1;
    switch (variant) {
        case 2: return launch_fmha<T, 1, 8>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, stream);
        case 3: return launch_fmha_pingpong<T>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, stream);
        default: return launch_fmha<T, 1, 4>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, stream);
    }
}

hipError_t fmha_fwd_dispatch(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                             int Sq, int Sk, float scale, int causal, int kv_valid_len, const FmhaStrides& sd, int dtype,
                             int variant, const FmhaWorkspace& ws, hipStream_t stream) {
    if (dtype == MI355_DTYPE_BF16)
        return fmha_fwd_dispatch_t<bf16_t>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, variant, ws, stream);
    return fmha_fwd_dispatch_t<half_t>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, variant, ws, stream);
}

}  // namespace mi355
