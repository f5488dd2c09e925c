// Fused multi-head attention forward for gfx950 (MI355X), head_dim 128, fp16 in/out, fp32 softmax statistics.
//
// Replaces the reference's attention ladder (kernels/fmha/pkg/fmha_unified/csrc/{auto,semi}/fmha_*.{cu,cpp});
// semantics follow semi/fmha_2_amd.cpp: BHSD layout (:33-45), kv head = q head / (Hq/Hkv), causal rule
// "masked iff q_pos < k_pos" (:187-190), keys at or beyond the valid length masked (:191, with the off-by-one
// of the reference corrected), scale 1/sqrt(d) supplied by the caller (:320).
//
// One kernel family, fmha_fwd_pingpong_kernel<T, QB> (8 phase-locked waves per workgroup, MFMA 16x16x32; 256 or 128 queries
// per workgroup), described at its definition. Everything stays in registers between the two matrix products:
//   S^T = K * Q^T      A operand = K fragment read from LDS (ds_read_b128), B operand = Q fragment held in registers for the
//                      whole kernel. A lane then owns ONE query column per 16-query block and 4 of the 16 keys of a key
//                      block, so the softmax statistics m, l and the rescale factor are per-lane scalars.
//   P^T                exp2((S - m) * scale*log2e) in fp32, rounded to fp16; the accumulator layout of S^T is (up to a
//                      fixed permutation of the keys) the B-operand layout of the second product, so P never leaves the
//                      registers.
//   O^T += V^T * P^T   A operand = V^T fragment, read from the row-major V tile in LDS with the transposing
//                      ds_read_b64_tr_b16 in that same key order.
// K and V tiles (64 keys x 128 d) are copied global -> LDS with 16-byte direct-to-LDS copies, double buffered,
// 16-byte chunks XOR-swizzled so that both the b128 reads (K) and the transposing reads (V) are conflict free.
#include <type_traits>
#include "mi355_common.h"
#include "mi355_serving_internal.h"
#include "mi355_timeline.h"

namespace mi355 {

// profiling build: per workgroup [wall: entry, loop start, loop end, exit; cycles: loop start, loop end; key tiles; 0]
MI355_TL(static __device__ unsigned long long fmha_fwd_stamps[timeline::kMaxWorkgroups * timeline::kSlots];)

namespace fmha {

constexpr int D = 128;            // head dim
constexpr int BN = 64;            // keys per tile
constexpr int ROW_BYTES = D * 2;  // 256
constexpr int TILE_BYTES = BN * ROW_BYTES;  // 16 KiB
constexpr float kLazyLog2 = 8.f;  // rescale only when a row maximum grows by more than 2^8

__device__ __forceinline__ int swz_k(int row) { return row & 15; }
__device__ __forceinline__ int swz_v16(int row) { return (row & 7) << 1; }   // 8 key rows x 32 bytes on distinct bank groups

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// maximum / sum over the four lanes that share l % 16
__device__ __forceinline__ float quad_max(float x) {
    x = fmaxf(x, __shfl_xor(x, 16, 64));
    return fmaxf(x, __shfl_xor(x, 32, 64));
}
__device__ __forceinline__ float quad_sum(float x) {
    x += __shfl_xor(x, 16, 64);
    return x + __shfl_xor(x, 32, 64);
}
// max(a, b, c) as one instruction. fmaxf() makes the compiler quiet possible signalling NaNs first (one extra
// v_max_f32 x, x per input); scores are never NaN here, and v_max3_f32 returns the non-NaN operands anyway.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

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

// ---------------------------------------------------------------------------------------------------------
// Ping-pong kernel: 8 waves x 32 queries per workgroup, two waves per SIMD that alternate roles. A wave alternates between
//     a matrix phase : S(j+1) = K(j+1) Q^T and O += V(j)^T P(j)      (matrix pipe + LDS reads)
//     a softmax phase: S(j+1) -> P(j+1)                               (VALU only)
// separated by workgroup barriers. Waves 4..7 run one phase behind waves 0..3, so on every SIMD one wave is in its matrix
// phase while the other is in its softmax phase: the matrix pipe and the VALU are busy at the same time without relying on
// the instruction scheduler to interleave them inside one wave. The phases of the workgroup are numbered P0, P1, ...; waves
// 0..3 run the matrix phase in the even ones, waves 4..7 in the odd ones. K and V have separate double buffers: tile j lives
// in Kbuf[j&1] / Vbuf[j&1], is copied by all 8 waves in an even phase (K(i+1) and V(i) at P(2i)) and has two phases to land
// (waited for at the end of P(2i+1)).
//
// Every product is made of MFMA 16x16x32 blocks: under the board's power limit that instruction sustains a ~14 % higher
// rate than 32x32x16 on random data (it also takes more VALU issue slots away from the partner wave's softmax, which is why
// the softmax below is cut down to the fewest instructions). Per wave and key tile (64 keys):
//   S^T[kb][qb] (16 keys x 16 queries) = K[kb] Q[qb]^T      4 key blocks x 2 query blocks x 4 steps of 32 d = 32 MFMAs
//   O^T[db][qb] (16 d x 16 queries)   += V[j]^T[db] P[j][qb]^T   8 d blocks x 2 query blocks x 2 steps of 32 keys = 32 MFMAs
//   l[qb]                             += 1 P[j][qb]^T            the softmax row sums, as a ninth all-ones "d block"  = 4 MFMAs
// Lane l = 16 g + c holds, of S^T[kb][qb], keys 16 kb + 4 g + 0..3 of query 16 qb + c. The B operand of the second
// product wants 8 keys of one query per lane: the four values of block 2j and the four of block 2j + 1 are taken as they
// lie, i.e. contraction index 8 g + i of step j stands for key 32 j + 4 g + i (i < 4) or 32 j + 16 + 4 g + (i - 4); the
// V^T fragment is gathered in that same order by two transposing LDS reads (key rows 32 j + 4 g .. and 32 j + 16 + 4 g ..),
// so P never leaves the registers. The softmax statistics of a query live in the 4 lanes c, c + 16, c + 32, c + 48; they
// only talk to each other when the running reference has to move (see the lazy rescaling below), which after the first
// tile is rare: the common path has no cross-lane operation at all.
// ---------------------------------------------------------------------------------------------------------
// QB = query blocks of 16 per wave: 2 (256 queries per workgroup) or 1 (128 queries, for shapes with too few 256-query
// workgroups to fill the machine and for short sequences; every K / V fragment then feeds one MFMA instead of two, and
// the kernel is held to 128 registers so that two workgroups share a CU).
template <typename T, int QB>
__global__ __launch_bounds__(512, (QB == 1 ? 4 : 2)) void fmha_fwd_pingpong_kernel(const T* __restrict__ Q, const T* __restrict__ K,
                                                               const T* __restrict__ V, T* __restrict__ O,
                                                               float* __restrict__ LSE, int B, int Hq, int Hkv, int Sq,
                                                               int Sk, float scale_log2, int causal, int kv_valid,
                                                               int q_tiles, FmhaStrides sd) {
    using namespace fmha;
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    constexpr int NWAVES = 8;
    constexpr int WQ = 16 * QB;          // queries per wave
    constexpr int BM = NWAVES * WQ;
    constexpr int COPIES = (BN * ROW_BYTES / 1024) / NWAVES;  // 2 wave-instructions per tile per wave

    MI355_TL(unsigned long long tl_w[4] = {timeline::wall_clock(), 0, 0, 0}; unsigned long long tl_c[2] = {0, 0};)
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;
    MI355_LDS char* kbuf = smem;                   // 2 x TILE_BYTES
    MI355_LDS char* vbuf = smem + 2 * TILE_BYTES;  // 2 x TILE_BYTES

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int late = wave >> 2;  // 0: waves 0..3 (matrix phase in even phases), 1: waves 4..7 (one phase behind)
    const int g = lane >> 4;
    const int c16 = lane & 15;

    int b, hq, q_tile;
    const int group = Hq / Hkv;
    fmha_decode_block(blockIdx.x, q_tiles, group, Hkv, B, b, hq, q_tile);
    const int hkv = hq / group;
    const int q_block0 = q_tile * BM;
    const int q_wave0 = q_block0 + wave * WQ;
    const int shift = Sk - Sq;

    const T* Qh = Q + b * sd.q_batch + hq * sd.q_head;
    const T* Kh = K + b * sd.k_batch + hkv * sd.k_head;
    const T* Vh = V + b * sd.v_batch + hkv * sd.v_head;
    T* Oh = O + b * sd.o_batch + hq * sd.o_head;

    int k_end = kv_valid;
    if (causal) k_end = min(k_end, min(q_block0 + BM, Sq) - 1 + shift + 1);
    const int n_tiles = (k_end + BN - 1) / BN;  // may be <= 0: no visible key for the whole workgroup

    // Q fragments (B operand of the first product): lane holds Q[16 qb + c][32 ks + 8 g .. +7]
    V8 qf[QB][4];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const int qrow = min(q_wave0 + qb * 16 + c16, Sq - 1);
        const T* qp = Qh + qrow * sd.q_row + 8 * g;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) qf[qb][ks] = *(const V8*)(qp + ks * 32);
    }

    // copy i of this wave covers tile rows 32 i + 4 wave + lane/16, 16-byte chunk position lane%16 (the swizzles depend on
    // row % 16 only, so both copies of a lane share their column offsets); rows past the last valid key are clamped onto
    // it (masked later, but V must not feed NaNs into 0 * V)
    const int copy_row0 = wave * 4 + (lane >> 4);
    const uint32_t copy_kcol = ((lane & 15) ^ swz_k(copy_row0)) * 16;
    const uint32_t copy_vcol = ((lane & 15) ^ swz_v16(copy_row0)) * 16;
    const uint32_t k_row_bytes = (uint32_t)sd.k_row * 2, v_row_bytes = (uint32_t)sd.v_row * 2;
    auto issue_k = [&](int tile) {
        const char* base = (const char*)Kh + (long)tile * BN * sd.k_row * 2;
        const int last = kv_valid - 1 - tile * BN;
#pragma unroll
        for (int i = 0; i < COPIES; ++i)
            copy16_global_to_lds(base, (uint32_t)min(copy_row0 + 32 * i, last) * k_row_bytes + copy_kcol,
                                 kbuf + (tile & 1) * TILE_BYTES + (i * NWAVES + wave) * 1024);
    };
    auto issue_v = [&](int tile) {
        const char* base = (const char*)Vh + (long)tile * BN * sd.v_row * 2;
        const int last = kv_valid - 1 - tile * BN;
#pragma unroll
        for (int i = 0; i < COPIES; ++i)
            copy16_global_to_lds(base, (uint32_t)min(copy_row0 + 32 * i, last) * v_row_bytes + copy_vcol,
                                 vbuf + (tile & 1) * TILE_BYTES + (i * NWAVES + wave) * 1024);
    };

    // K fragment (key block kb, d step ks): row 16 kb + c, chunk (4 ks + g) ^ (row & 15)
    const int k_base = c16 * ROW_BYTES + ((g ^ c16) << 4);                 // xor (ks << 6), + kb * 16 * ROW_BYTES
    // V^T fragment (key step j, d block db), transposing read t: input lane c of a 16-lane group supplies 4 d of key row
    // 32 j + 16 t + 4 g + c / 4: d 16 db + 4 (c % 4) .. +3
    const int v_row = 4 * g + (c16 >> 2);
    const int v_base = v_row * ROW_BYTES + (((((c16 & 3) >> 1)) ^ swz_v16(v_row)) << 4) + (c16 & 1) * 8;   // xor (db << 5)

    float4v o[8][QB];
#pragma unroll
    for (int db = 0; db < 8; ++db)
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) o[db][qb] = float4v{0.f, 0.f, 0.f, 0.f};
    // Row sums of P ride on the matrix pipe: a ninth "d block" whose V^T rows are all ones, l[qb] += 1 P[j][qb]^T. Every
    // row of that block (so all four elements of a lane) ends up holding the sum over all keys of the lane's query,
    // accumulated from the same fp16-rounded P the output uses; no VALU additions and no cross-lane sum are needed.
    // The rounding of P enters l with a relative error of at most 2^-12 for fp16, far inside the 1e-3 allowed on the
    // log-sum-exp; for bfloat16 (2^-9) it would not be, so that type sums the unrounded fp32 values on the VALU instead
    // (element 0 of l_acc then holds this lane's partial sum; the four lanes of a query are added at the end).
    constexpr bool kSumOnMatrixPipe = std::is_same<T, half_t>::value;
    float4v l_acc[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) l_acc[qb] = float4v{0.f, 0.f, 0.f, 0.f};
    V8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (T)1.0f;
    float m_run[QB];
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) m_run[qb] = -INFINITY;

    // empty asm statements that make a value "used" at a program point: they keep the softmax in its phase and the MFMAs
    // in theirs (the compiler is otherwise free to move register-only work across s_barrier)
    auto pin_s = [](float4v(&s)[4][QB]) {
        if constexpr (QB == 2)
            asm volatile("" : "+v"(s[0][0]), "+v"(s[0][1]), "+v"(s[1][0]), "+v"(s[1][1]), "+v"(s[2][0]), "+v"(s[2][1]), "+v"(s[3][0]), "+v"(s[3][1]));
        else
            asm volatile("" : "+v"(s[0][0]), "+v"(s[1][0]), "+v"(s[2][0]), "+v"(s[3][0]));
    };
    auto pin_p = [](V8(&pf)[2][QB]) {
        if constexpr (QB == 2) asm volatile("" : "+v"(pf[0][0]), "+v"(pf[0][1]), "+v"(pf[1][0]), "+v"(pf[1][1]));
        else asm volatile("" : "+v"(pf[0][0]), "+v"(pf[1][0]));
    };
    auto pin_o = [&]() {
        if constexpr (QB == 2) {
            asm volatile("" : "+v"(l_acc[0]), "+v"(l_acc[1]));
#pragma unroll
            for (int db = 0; db < 8; db += 4)
                asm volatile("" : "+v"(o[db][0]), "+v"(o[db][1]), "+v"(o[db + 1][0]), "+v"(o[db + 1][1]), "+v"(o[db + 2][0]), "+v"(o[db + 2][1]),
                                  "+v"(o[db + 3][0]), "+v"(o[db + 3][1]));
        } else {
            asm volatile("" : "+v"(l_acc[0]), "+v"(o[0][0]), "+v"(o[1][0]), "+v"(o[2][0]), "+v"(o[3][0]), "+v"(o[4][0]), "+v"(o[5][0]), "+v"(o[6][0]),
                              "+v"(o[7][0]));
        }
    };

    int phase = 0;  // index of the workgroup phase this wave is in
    bool copies_due = false;
    auto next_phase = [&]() {
        if (phase & 1) wait_vmcnt<0>();  // copies issued at the start of the previous (even) phase have landed
        __syncthreads();
        ++phase;
        if (!(phase & 1)) {
            if (!late) { copies_due = true; return; }   // a wave entering its matrix phase issues them behind its first reads
            const int i = phase >> 1;
            if (i + 1 < n_tiles) issue_k(i + 1);
            if (i < n_tiles) issue_v(i);
        }
    };
    auto due_copies = [&]() {
        if (copies_due) {
            copies_due = false;
            const int i = phase >> 1;
            if (i + 1 < n_tiles) issue_k(i + 1);
            if (i < n_tiles) issue_v(i);
        }
    };

    // Fragment f of a matrix phase, in the order the MFMAs consume them: f < 16 is the K fragment (ks = f / 4, kb = f % 4),
    // f >= 16 the V^T fragment (j = (f - 16) / 8, db = (f - 16) % 8). Each fragment feeds two MFMAs (the two query blocks).
    auto read_frag = [&](MI355_LDS char* kst, MI355_LDS char* vst, int f) -> V8 {
        if (f < 16) {
            const int ks = f >> 2, kb = f & 3;
            return Elem<T>::frag(lds_read_b128(kst + ((k_base ^ (ks << 6)) + kb * 16 * ROW_BYTES)));
        }
        const int j = (f - 16) >> 3, db = (f - 16) & 7;
        const int off = (v_base ^ (db << 5)) + (32 * j) * ROW_BYTES;
        return Elem<T>::frag(concat(lds_read_tr16_b64(vst + off), lds_read_tr16_b64(vst + off + 16 * ROW_BYTES)));
    };
    // The matrix phase over fragments [F0, F1): every fragment is read AHEAD fragments (12 MFMAs, 192 cycles) ahead of its
    // MFMAs, into the register its predecessor has just released; sched_barrier pins that order.
    auto mfma_phase = [&](auto f0c, auto f1c, int tile_k, float4v(&s)[4][QB], int tile_v, const V8(&pf)[2][QB]) {
        constexpr int F0 = decltype(f0c)::value, F1 = decltype(f1c)::value;
        MI355_LDS char* kst = kbuf + (tile_k & 1) * TILE_BYTES;
        MI355_LDS char* vst = vbuf + (tile_v & 1) * TILE_BYTES;
        constexpr int AHEAD = QB == 1 ? 5 : 6;
        V8 fr[AHEAD];
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) fr[i] = read_frag(kst, vst, F0 + i);
        due_copies();
        if constexpr (F0 == 0) {
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[kb][qb] = float4v{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int f = F0; f < F1; ++f) {
            __builtin_amdgcn_sched_barrier(0);
            const int r = (f - F0) % AHEAD;
            if (f < 16) {
                const int ks = f >> 2, kb = f & 3;
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[kb][qb] = Elem<T>::mfma16(fr[r], qf[qb][ks], s[kb][qb]);
            } else {
                const int j = (f - 16) >> 3, db = (f - 16) & 7;
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) o[db][qb] = Elem<T>::mfma16(fr[r], pf[j][qb], o[db][qb]);
                if (kSumOnMatrixPipe && db == 3) {   // the row sums of this key step, in the middle of its eight d blocks
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb) l_acc[qb] = Elem<T>::mfma16(ones, pf[j][qb], l_acc[qb]);
                }
            }
            if (f + AHEAD < F1) fr[r] = read_frag(kst, vst, f + AHEAD);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I16 = std::integral_constant<int, 16>;
    using I32 = std::integral_constant<int, 32>;

    auto softmax_tile = [&](float4v(&s)[4][QB], int tile, V8(&pf)[2][QB]) {
        const int key0 = tile * BN;
        const bool need_mask = (key0 + BN > kv_valid) || (causal && (key0 + BN - 1 > q_wave0 + shift));
        if (need_mask) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                const int qi = q_wave0 + qb * 16 + c16;
                const int lim = causal ? min(kv_valid - 1, qi + shift) : kv_valid - 1;  // last visible key
#pragma unroll
                for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (key0 + kb * 16 + 4 * g + e > lim) s[kb][qb][e] = -INFINITY;
            }
        }
        // Lazy rescaling: m_run is the exponent reference of the running sums of a query (identical in its four lanes), not
        // necessarily its running maximum. A lane only asks for it to move when one of ITS scores exceeds it by more than
        // 2^kLazyLog2; then (any lane of the wave asked) the four lanes of every query agree on the tile's maximum and the
        // reference is raised to the running maximum. Otherwise P = exp2((S - m_run) c) <= 2^kLazyLog2 everywhere and nothing
        // crosses lanes.
        float mx[QB];
        bool raise = false;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            float a = max3(s[0][qb][0], s[0][qb][1], s[0][qb][2]);
            float c = max3(s[0][qb][3], s[1][qb][0], s[1][qb][1]);
            a = max3(a, s[1][qb][2], s[1][qb][3]);
            c = max3(c, s[2][qb][0], s[2][qb][1]);
            a = max3(a, s[2][qb][2], s[2][qb][3]);
            c = max3(c, s[3][qb][0], s[3][qb][1]);
            a = max3(a, s[3][qb][2], s[3][qb][3]);
            a = max3(a, c, c);
            mx[qb] = a;
            raise = raise || ((a - m_run[qb]) * scale_log2 > kLazyLog2);  // -inf - -inf = NaN compares false
        }
        if (__builtin_amdgcn_ballot_w64(raise) != 0) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                const float m_new = fmaxf(m_run[qb], quad_max(mx[qb]));
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = fast_exp2((m_run[qb] - m_use) * scale_log2);
                m_run[qb] = m_new;
#pragma unroll
                for (int e = 0; e < 4; ++e) l_acc[qb][e] *= alpha;
#pragma unroll
                for (int db = 0; db < 8; ++db)
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[db][qb][e] *= alpha;
            }
        }
        // the wave is the only one of its SIMD issuing VALU work in this phase, so dependent instructions are kept apart:
        // all multiply-adds, then all exponentials, then the sums and conversions
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const float neg_ms = (m_run[qb] == -INFINITY) ? 0.f : -m_run[qb] * scale_log2;
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                for (int e = 0; e < 4; ++e) s[kb][qb][e] = __builtin_fmaf(s[kb][qb][e], scale_log2, neg_ms);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < 4; ++kb)
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int e = 0; e < 4; ++e) s[kb][qb][e] = fast_exp2(s[kb][qb][e]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            float ps[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                V8 pk;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (!kSumOnMatrixPipe) ps[e] += s[2 * j][qb][e] + s[2 * j + 1][qb][e];
                    pk[e] = (T)s[2 * j][qb][e];
                    pk[4 + e] = (T)s[2 * j + 1][qb][e];
                }
                pf[j][qb] = pk;
            }
            if (!kSumOnMatrixPipe) l_acc[qb][0] += (ps[0] + ps[1]) + (ps[2] + ps[3]);
        }
    };

    if (n_tiles > 0) {
        // before P0: K(0) must be in LDS
        issue_k(0);
        wait_vmcnt<0>();
        __syncthreads();
        if (1 < n_tiles) issue_k(1);  // start of P0
        issue_v(0);
        if (late) next_phase();  // waves 4..7 idle during P0

        float4v s[4][QB];
        V8 pf[2][QB];
        MI355_TL(tl_w[1] = timeline::wall_clock(); tl_c[0] = timeline::shader_cycles();)
        __builtin_amdgcn_s_setprio(1);
        mfma_phase(I0{}, I16{}, 0, s, 0, pf);               // S(0) alone
        __builtin_amdgcn_s_setprio(0);
        pin_s(s);
        next_phase();
        for (int j = 0; j + 1 < n_tiles; ++j) {
            softmax_tile(s, j, pf);
            pin_p(pf);
            next_phase();
            __builtin_amdgcn_s_setprio(1);
            mfma_phase(I0{}, I32{}, j + 1, s, j, pf);        // S(j+1) and O += V(j)^T P(j)
            __builtin_amdgcn_s_setprio(0);
            pin_s(s);
            pin_o();
            next_phase();
        }
        softmax_tile(s, n_tiles - 1, pf);
        pin_p(pf);
        next_phase();
        mfma_phase(I16{}, I32{}, 0, s, n_tiles - 1, pf);     // O += V(last)^T P(last) alone
        next_phase();
        if (!late) next_phase();  // waves 0..3 idle while waves 4..7 finish
    }
    MI355_TL(tl_w[2] = timeline::wall_clock(); tl_c[1] = timeline::shader_cycles();)

    // ---- finalize: O / l, LSE: lane holds O[query 16 qb + c][d = 16 db + 4 g + 0..3] -----------------------------
#pragma unroll
    for (int qb = 0; qb < QB; ++qb) {
        const float l_tot = kSumOnMatrixPipe ? l_acc[qb][0] : quad_sum(l_acc[qb][0]);
        const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
        const int qi = q_wave0 + qb * 16 + c16;
        if (qi < Sq) {
            T* orow = Oh + qi * sd.o_row + 4 * g;
#pragma unroll
            for (int db = 0; db < 8; ++db) {
                V4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (T)(o[db][qb][e] * inv);
                *(V4*)(orow + db * 16) = v;
            }
            if (LSE != nullptr && g == 0) {
                const float lse = (l_tot > 0.f) ? (m_run[qb] * scale_log2 + __builtin_log2f(l_tot)) * 0.69314718055994531f : -INFINITY;
                LSE[((long)b * Hq + hq) * (long)Sq + qi] = lse;
            }
        }
    }
    MI355_TL(
        wait_vmcnt<0>();   // the stores of this wave have been accepted
        tl_w[3] = timeline::wall_clock();
        if (tid == 0 && blockIdx.x < timeline::kMaxWorkgroups) {
            unsigned long long* rec = fmha_fwd_stamps + (long)blockIdx.x * timeline::kSlots;
            rec[0] = tl_w[0]; rec[1] = tl_w[1]; rec[2] = tl_w[2]; rec[3] = tl_w[3];
            rec[4] = tl_c[0]; rec[5] = tl_c[1]; rec[6] = (unsigned long long)max(n_tiles, 0); rec[7] = 0;
        })
}

template <typename T, int QB>
static hipError_t launch_fmha_pingpong(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq,
                                       int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd,
                                       hipStream_t stream) {
    constexpr int BM = 128 * QB;
    constexpr int LDS = 4 * fmha::TILE_BYTES;
    auto kern = fmha_fwd_pingpong_kernel<T, QB>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), LDS); e != hipSuccess) return e;
    const int q_tiles = (Sq + BM - 1) / BM;
    const long blocks = (long)q_tiles * Hq * B;
    if (blocks > 0x7fffffffL) return hipErrorInvalidValue;
    const float scale_log2 = scale * 1.4426950408889634f;
    kern<<<dim3((unsigned)blocks), dim3(512), LDS, stream>>>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale_log2, causal, kv_valid,
                                                             q_tiles, sd);
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
    // the kernels address a K/V tile with 32-bit byte offsets from its first row
    if (sd.k_row >= (1L << 24) || sd.v_row >= (1L << 24)) return hipErrorNotSupported;
    if (variant == 0 && fmha_decode_applicable(B, Hq, Hkv, Sq, Sk, kv_valid_len))
        return fmha_decode_dispatch<T>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, ws, stream);
    if (variant == 0) {
        // 256-query workgroups once there are clearly more of them than CUs (with exactly one per CU a causal problem runs
        // as long as its heaviest tile; 128-query workgroups then balance better and still fill the machine) and the
        // sequences are long enough to amortise their longer prologue. Measured (b, heads 32/8, s, 128- vs 256-query):
        // 1 x 1024 causal 25 / 35 us, 1 x 2048 57 / 65, 8 x 512 43 / 50, 1 x 3000 108 / 94, 1 x 4096 182 / 144,
        // 4 x 1024 (32 kv heads, non-causal) 100 / 82.
        // A causal problem whose keys are its own queries computes every diagonal block in full: with 256-query workgroups
        // that is 1 / (2 Sq / 256) more work than with 128-query ones, which outweighs their cheaper inner loop below
        // ~1400 queries (many workgroups either way; 128- / 256-query: 16 x 768 127 / 136 us, 8 x 1024 101 / 108,
        // 8 x 1280 142 / 146, 4 x 1536 101 / 99, 4 x 2048 169 / 153).
        const long wg256 = (long)((Sq + 255) / 256) * Hq * B;
        const bool diagonal_heavy = causal && Sk < 2L * Sq;
        variant = (wg256 >= 320 && Sq > (diagonal_heavy ? 1408 : 512)) ? 2 : 1;
    }
    if (variant == 2) return launch_fmha_pingpong<T, 2>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, stream);
    return launch_fmha_pingpong<T, 1>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, stream);
}

hipError_t fmha_fwd_dispatch(const void* Q, const void* K, const void* V, void* O, float* LSE, int B, int Hq, int Hkv,
                             int Sq, int Sk, float scale, int causal, int kv_valid_len, const FmhaStrides& sd, int dtype,
                             int variant, const FmhaWorkspace& ws, hipStream_t stream) {
    if (dtype == MI355_DTYPE_BF16)
        return fmha_fwd_dispatch_t<bf16_t>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, variant, ws, stream);
    return fmha_fwd_dispatch_t<half_t>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, variant, ws, stream);
}

}  // namespace mi355

#ifdef MI355_TIMELINE
// profiling build: copies the records of the last attention forward launch (kMaxWorkgroups x kSlots 64-bit values) to the host
extern "C" int mi355_timeline_read_fmha_fwd(void* dst, size_t bytes) {
    const size_t all = sizeof(unsigned long long) * mi355::timeline::kMaxWorkgroups * mi355::timeline::kSlots;
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(mi355::fmha_fwd_stamps), bytes < all ? bytes : all);
}
#endif
