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
// K and V tiles (64 keys x 128 d) are copied global -> LDS with 16-byte direct-to-LDS copies into a ring of four slots
// per operand, 16-byte chunks XOR-swizzled so that both the b128 reads (K) and the transposing reads (V) are conflict free.
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
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
// Register (index into the AHEAD fragment registers) of the i-th fragment of a matrix phase when fragments are read in
// order and consumed pairwise swapped (1, 0, 3, 2, ..): fragment i >= AHEAD goes where the fragment consumed just before its
// read was, i.e. where fragment (i - AHEAD) ^ 1 lived.
__device__ __forceinline__ constexpr int frag_reg(int i, int ahead) { return i < ahead ? i : frag_reg((i - ahead) ^ 1, ahead); }
// the same, kept in program order relative to its like
__device__ __forceinline__ float max3v(float a, float b, float c) {
    float r;
    asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

}  // namespace fmha

// Work item `round` of workgroup `wg` out of `n_wg`: a (batch, q head, q tile), or false when the workgroup has none left.
// A launch has at most one workgroup per CU; each walks its own list of items (no global counter: nothing to reset, nothing
// two launches could share). Workgroups with ids congruent mod 8 share an XCD (and its L2): when the (batch, kv head)
// groups divide evenly every XCD gets whole groups, so K and V are fetched from HBM once. On an XCD the items are ranked
// with the q tiles that see the most keys (causal) first and dealt out in rounds that run forwards and backwards in turn:
// the workgroup that got the heaviest item of one round gets the lightest of the next.
__device__ __forceinline__ bool fmha_work_item(int wg, int n_wg, int round, int q_tiles, int group, int Hkv, int B, int& b,
                                               int& hq, int& q_tile) {
    const int kv_groups = Hkv * B;
    int x = 0, n_x = 1;
    if (kv_groups % 8 == 0 && n_wg % 8 == 0) {
        x = wg % 8;
        n_x = 8;
    }
    const int wl = wg / n_x, wgs = n_wg / n_x;   // workgroup index on its XCD, workgroups per XCD
    const int gpx = kv_groups / n_x;             // (batch, kv head) groups per XCD
    const int per_rank = gpx * group;            // items of one q tile on this XCD
    const int u = round * wgs + ((round & 1) ? wgs - 1 - wl : wl);
    if (u >= per_rank * q_tiles) return false;
    const int rank = u / per_rank, rem = u - rank * per_rank;
    const int gl = rem / group, hin = rem - gl * group;
    q_tile = q_tiles - 1 - rank;
    const int kvg = x * gpx + gl;
    b = kvg / Hkv;
    hq = (kvg - b * Hkv) * group + hin;
    return true;
}

// ---------------------------------------------------------------------------------------------------------
// Ping-pong kernel: 8 waves x 16 QB queries per workgroup, two waves per SIMD that alternate roles. A wave alternates between
//     a matrix phase : S(j+1) = K(j+1) Q^T and O += V(j)^T P(j)      (matrix pipe + LDS reads)
//     a softmax phase: S(j+1) -> P(j+1)                               (VALU; the tile copies ride along)
// separated by workgroup barriers. Waves 4..7 run one phase behind waves 0..3, so on every SIMD one wave is in its matrix
// phase while the other is in its softmax phase: the matrix pipe and the VALU are busy at the same time without relying on
// the instruction scheduler to interleave them inside one wave. The phases of the workgroup are numbered P0, P1, ...; waves
// 0..3 run the matrix phase in the even ones, waves 4..7 in the odd ones.
//
// Every product is made of MFMA 16x16x32 blocks: under the board's power limit that instruction sustains a ~14 % higher
// rate than 32x32x16 on random data. Per wave and key tile (64 keys), QB = 2:
//   S^T[kb][qb] (16 keys x 16 queries) = K[kb] Q[qb]^T      4 key blocks x 2 query blocks x 4 steps of 32 d = 32 MFMAs
//   O^T[db][qb] (16 d x 16 queries)   += V[j]^T[db] P[j][qb]^T   8 d blocks x 2 query blocks x 2 steps of 32 keys = 32 MFMAs
//   l[qb]                             += 1 P[j][qb]^T            the softmax row sums, as a ninth all-ones "d block"  = 4 MFMAs
// Lane l = 16 g + c holds, of S^T[kb][qb], keys 16 kb + 4 g + 0..3 of query 16 qb + c. The B operand of the second
// product wants 8 keys of one query per lane: the four values of block 2j and the four of block 2j + 1 are taken as they
// lie, i.e. contraction index 8 g + i of step j stands for key 32 j + 4 g + i (i < 4) or 32 j + 16 + 4 g + (i - 4); the
// V^T fragment is gathered in that same order by two transposing LDS reads (key rows 32 j + 4 g .. and 32 j + 16 + 4 g ..),
// so P never leaves the registers. The softmax statistics of a query live in the 4 lanes c, c + 16, c + 32, c + 48; they
// only talk to each other when the running reference has to move (lazy rescaling, below), which after the first tile is
// rare: the common path has no cross-lane operation at all.
//
// A wave issues about one instruction per 5 cycles when it has its SIMD to itself and one per 10-12 next to the partner
// wave's MFMAs, whatever the instruction is (scalar bookkeeping included): the phases are bound by their instruction
// COUNT, and the loop is built to need few:
//   * The K / V tiles live in a ring of NBUF = 4 slots per operand and the main loop is unrolled four times, so every LDS
//     address of a fragment read is a loop-invariant register plus an immediate offset (no address arithmetic in the
//     matrix phase), and the LDS destination of a copy is an immediate added into M0.
//   * A tile pair {K(q), V(q-1)} (read in the phases P(2q) and P(2q+1)) is copied by every wave during its softmax phase
//     three tile steps earlier, one copy instruction between two blocks of VALU work (issued together right behind a
//     barrier, the 32 copy instructions of a pair queue up in the CU's memory pipeline and hold every wave at its issue for
//     ~450 cycles). In the unrolled loop all 64 rows of the tile exist, so a copy is three instructions (M0, wait state,
//     load: the tile base is a scalar pointer that advances once per tile, the lane offset a loop-invariant register); the
//     last few tiles of a workgroup run a general loop whose copies clamp the tile index and the row.
//   * The pair is published (s_waitcnt vmcnt + barrier) at the end of P(2q-2), a whole phase before its first use, so a
//     wave reads the first fragments of its next matrix phase at the end of its softmax phase, in front of the barrier, and
//     the matrix pipe starts on operands that are already in registers.
//   * The softmax keeps, per query, the threshold that makes the exponent reference move and the negated scaled reference
//     as state (recomputed only when the reference moves): the common path is max tree, one compare, fma, exp2, pack.
// QB = query blocks of 16 per wave: 2 (256 queries per workgroup) or 1 (128 queries, for shapes with too few 256-query
// workgroups to fill the machine and for short sequences; every K / V fragment then feeds one MFMA instead of two).
// ---------------------------------------------------------------------------------------------------------
// 16-byte global -> LDS copy whose LDS address is a scalar register plus a compile-time constant (added straight into M0)
template <int IMM>
__device__ __forceinline__ void copy16_global_to_lds_at(const void* uniform_base, uint32_t lane_byte_offset, uint32_t lds_wave_base) {
    asm volatile(
        "s_add_u32 m0, %2, %3\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, %1"
        :
        : "v"(lane_byte_offset), "s"(uniform_base), "s"(lds_wave_base), "n"(IMM)
        : "memory", "m0", "scc");
}

// SEG: the keys are cut into `segments` ranges of seg_len keys (a multiple of 64) and a work item is (batch, range, head, q
// tile): it attends to its range only (K and V start seg * seg_len rows further on, the valid length and the causal limit
// are counted from there) and writes its O, normalised over its range, and its LSE to the partial buffers
// O [segments][B][Hq][Sq][128] and LSE [segments][B][Hq][Sq]; fmha_merge_segments_kernel combines them. For a few queries
// against a long cache, where one item per (head, q tile) would leave most CUs idle behind a long walk over the keys.
template <typename T, int QB, bool SEG = false>
__global__ __launch_bounds__(512, 2) void fmha_fwd_pingpong_kernel(const T* __restrict__ Q, const T* __restrict__ K,
                                                               const T* __restrict__ V, T* __restrict__ O,
                                                               float* __restrict__ LSE, int B, int Hq, int Hkv, int Sq,
                                                               int Sk, float scale_log2, int causal, int kv_valid,
                                                               int q_tiles, FmhaStrides sd, int segments, int seg_len) {
    using namespace fmha;
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    constexpr int NWAVES = 8;
    constexpr int NBUF = 4;
    constexpr int WQ = 16 * QB;          // queries per wave
    constexpr int BM = NWAVES * WQ;
    constexpr int VBUF0 = NBUF * TILE_BYTES;   // LDS: NBUF K slots, then NBUF V slots; slot q % NBUF holds K(q) and V(q - 1)
    static_assert(BN * ROW_BYTES / 1024 / NWAVES == 2, "the softmax phase carries four copy slots: two of K, two of V");

    MI355_TL(unsigned long long tl_w[4] = {timeline::wall_clock(), 0, 0, 0}; unsigned long long tl_c[2] = {0, 0};)
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int late = wave >> 2;  // 0: waves 0..3 (matrix phase in even phases), 1: waves 4..7 (one phase behind)
    const int g = lane >> 4;
    const int c16 = lane & 15;

    // ---- the work item this workgroup is on (set_item) --------------------------------------------------------------
    const int group = Hq / Hkv;
    int shift = Sk - Sq;
    const int kv_valid_all = kv_valid;
    long o_row = sd.o_row;
    int b = 0, hq = 0, q_wave0 = 0, n_tiles = 0, n_full = 0, last_tile = 0;
    const T* Qh = Q;
    const T* Kh = K;
    const T* Vh = V;
    T* Oh = O;
    auto set_item = [&](int round) -> bool {
        int q_tile;
        if (!fmha_work_item(blockIdx.x, gridDim.x, round, q_tiles, group, Hkv, SEG ? B * segments : B, b, hq, q_tile)) return false;
        const int hkv = hq / group;
        const int q_block0 = q_tile * BM;
        q_wave0 = q_block0 + wave * WQ;
        if constexpr (SEG) {   // b counts (batch, range) pairs
            const int seg = b % segments;
            b /= segments;
            const long k0 = (long)seg * seg_len;
            Qh = Q + b * sd.q_batch + hq * sd.q_head;
            Kh = K + b * sd.k_batch + hkv * sd.k_head + k0 * sd.k_row;
            Vh = V + b * sd.v_batch + hkv * sd.v_head + k0 * sd.v_row;
            Oh = O + (((long)seg * B + b) * Hq + hq) * (long)Sq * D;
            o_row = D;
            kv_valid = min(max(kv_valid_all - (int)k0, 0), seg_len);
            shift = Sk - Sq - (int)k0;
            b = seg * B + b;   // the LSE row of this item, below
        } else {
        Qh = Q + b * sd.q_batch + hq * sd.q_head;
        Kh = K + b * sd.k_batch + hkv * sd.k_head;
        Vh = V + b * sd.v_batch + hkv * sd.v_head;
        Oh = O + b * sd.o_batch + hq * sd.o_head;
        }
        int k_end = kv_valid;
        if (causal) k_end = min(k_end, min(q_block0 + BM, Sq) - 1 + shift + 1);
        n_tiles = (k_end + BN - 1) / BN;            // may be <= 0: no visible key for the whole work item
        n_full = min(n_tiles, kv_valid / BN);       // tiles 0 .. n_full-1 have all 64 rows
        last_tile = n_tiles - 1;
        return true;
    };

    // Q fragments (B operand of the first product): lane holds Q[16 qb + c][32 ks + 8 g .. +7]
    V8 qf[QB][4];
    auto load_q = [&]() {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const int qrow = min(q_wave0 + qb * 16 + c16, Sq - 1);
            const T* qp = Qh + qrow * sd.q_row + 8 * g;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qf[qb][ks] = *(const V8*)(qp + ks * 32);
        }
    };

    // copy i of this wave covers tile rows 32 i + 4 wave + lane/16, 16-byte chunk position lane%16
    const int copy_row0 = wave * 4 + (lane >> 4);
    const uint32_t copy_kcol = ((lane & 15) ^ swz_k(copy_row0)) * 16;
    const uint32_t copy_vcol = ((lane & 15) ^ swz_v16(copy_row0)) * 16;
    const uint32_t k_row_bytes = (uint32_t)sd.k_row * 2, v_row_bytes = (uint32_t)sd.v_row * 2;
    const long k_tile_bytes = (long)BN * sd.k_row * 2, v_tile_bytes = (long)BN * sd.v_row * 2;
    const uint32_t lds_wave = (uint32_t)(uintptr_t)smem + (uint32_t)wave * 1024u;
    // general copies: the tile index is clamped to the last tile (past the end a copy re-reads that tile into a slot nobody
    // reads any more) and rows past the last valid key onto it (masked later, but V must not feed NaNs into 0 * V)
    auto issue_k1 = [&](int q, int i) {   // half i of K(q) into slot q % NBUF
        const int tile = min(q, last_tile);
        const int last = kv_valid - 1 - tile * BN;
        copy16_global_to_lds((const char*)Kh + tile * k_tile_bytes, (uint32_t)min(copy_row0 + 32 * i, last) * k_row_bytes + copy_kcol,
                             smem + (q & (NBUF - 1)) * TILE_BYTES + (i * NWAVES + wave) * 1024);
    };
    auto issue_v1 = [&](int q, int i) {   // half i of V(q - 1) into slot q % NBUF
        const int tile = max(min(q - 1, last_tile), 0);
        const int last = kv_valid - 1 - tile * BN;
        copy16_global_to_lds((const char*)Vh + tile * v_tile_bytes, (uint32_t)min(copy_row0 + 32 * i, last) * v_row_bytes + copy_vcol,
                             smem + VBUF0 + (q & (NBUF - 1)) * TILE_BYTES + (i * NWAVES + wave) * 1024);
    };
    // copies of the unrolled loop: tile base pointers of K(j + 3) and V(j + 2), advanced once per tile step
    uint32_t k_lane_off[2], v_lane_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        k_lane_off[i] = (uint32_t)(copy_row0 + 32 * i) * k_row_bytes + copy_kcol;
        v_lane_off[i] = (uint32_t)(copy_row0 + 32 * i) * v_row_bytes + copy_vcol;
    }
    const char* k_next = nullptr;
    const char* v_next = nullptr;
    // the first pairs of the current item: K(0), K(1), V(0), K(2), V(1)
    auto issue_first_pairs = [&]() {
        issue_k1(0, 0); issue_k1(0, 1);
        issue_k1(1, 0); issue_k1(1, 1);
        issue_v1(1, 0); issue_v1(1, 1);
        issue_k1(2, 0); issue_k1(2, 1);
        issue_v1(2, 0); issue_v1(2, 1);
        k_next = (const char*)Kh + 3 * k_tile_bytes;
        v_next = (const char*)Vh + 2 * v_tile_bytes;
    };

    // fragment addresses: loop-invariant registers, the slot and the block inside the tile are immediate offsets
    //   K fragment (key block kb, d step ks): row 16 kb + c, chunk (4 ks + g) ^ (row & 15)
    //   V^T fragment (key step j, d block db), transposing read t: key row 32 j + 16 t + 4 g + c / 4, d 16 db + 4 (c % 4) .. +3
    MI355_LDS char* k_ptr[4];
    MI355_LDS char* v_ptr[8];
    {
        const int k_base = c16 * ROW_BYTES + ((g ^ c16) << 4);
        const int v_row = 4 * g + (c16 >> 2);
        const int v_base = v_row * ROW_BYTES + (((((c16 & 3) >> 1)) ^ swz_v16(v_row)) << 4) + (c16 & 1) * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) k_ptr[ks] = smem + (k_base ^ (ks << 6));
#pragma unroll
        for (int db = 0; db < 8; ++db) v_ptr[db] = smem + VBUF0 + (v_base ^ (db << 5));
    }

    float4v o[8][QB];
    constexpr bool kSumOnMatrixPipe = std::is_same<T, half_t>::value;
    float4v l_acc[QB];
    V8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = (T)1.0f;
    asm volatile("" : "+v"(ones));   // in vector registers for good (the compiler would re-materialise it in every matrix phase)
    // per query: exponent reference of the running sums, the score above which it has to move, and -reference * scale
    float m_run[QB], m_thr[QB], neg_ms[QB];
    const float lazy_margin = kLazyLog2 / scale_log2;

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

    // s_barrier as inline assembly: in front of a barrier it recognises the compiler waits for every LDS read it knows of,
    // and the fragments read ahead for the next matrix phase are meant to stay in flight across this one. Nothing else
    // crosses: the reads of a matrix phase have been consumed by its MFMAs, the copies are waited for explicitly.
    auto phase_barrier = []() { asm volatile("s_barrier" ::: "memory"); };
    // At the end of an even phase the pair of the step after next must have landed (all but this wave's four newest
    // copies), so that the barrier publishes it a whole phase ahead of its first reader. The same wait at the end of an odd
    // phase finds nothing to wait for (a wave's newest four copies are all that is outstanding there), so every phase ends
    // the same way and no wave has to know which half of the workgroup it belongs to.
    auto end_phase = [&]() { wait_vmcnt<4>(); phase_barrier(); };
    constexpr int AHEAD = 6;   // fragments in flight ahead of their MFMAs
    // fragment f of the matrix phase on the pair in ring slot `slot`: f < 16 K (ks = f / 4, kb = f % 4), f >= 16 V^T
    // (j = (f - 16) / 8, db = (f - 16) % 8); SLOT >= 0: compile-time slot, the whole offset is an immediate
    auto read_frag = [&](auto slot_c, int slot, int f) -> V8 {
        constexpr int SLOT = decltype(slot_c)::value;
        const int so = (SLOT >= 0 ? SLOT : slot) * TILE_BYTES;
        if (f < 16) {
            const int ks = f >> 2, kb = f & 3;
            return Elem<T>::frag(lds_read_b128(k_ptr[ks] + (so + kb * 16 * ROW_BYTES)));
        }
        const int j = (f - 16) >> 3, db = (f - 16) & 7;
        MI355_LDS char* p = v_ptr[db] + (so + (32 * j) * ROW_BYTES);
        return Elem<T>::frag(concat(lds_read_tr16_b64(p), lds_read_tr16_b64(p + 16 * ROW_BYTES)));
    };
    auto preload = [&](auto f0c, auto slot_c, int slot, V8(&fr)[AHEAD]) {
        constexpr int F0 = decltype(f0c)::value;
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) fr[i] = read_frag(slot_c, slot, F0 + i);
    };
    // matrix phase over fragments [F0, F1): S = K Q^T (f < 16) and O += V^T P (f >= 16); fr holds the first AHEAD fragments
    auto mfma_phase = [&](auto f0c, auto f1c, auto slot_c, int slot, float4v(&s)[4][QB], const V8(&pf)[2][QB], V8(&fr)[AHEAD]) {
        constexpr int F0 = decltype(f0c)::value, F1 = decltype(f1c)::value;
        if constexpr (F0 == 0) {
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[kb][qb] = float4v{0.f, 0.f, 0.f, 0.f};
        }
        // Fragments are read in the order f = F0, F0 + 1, .. and consumed in pairs, the later-read one first: LDS reads complete
        // in order, so the wait for it covers its predecessor and a pair costs one s_waitcnt instead of two. The register a
        // fragment frees takes the next fragment in read order (frag_reg).
        auto use = [&](int f) {
            const int r = frag_reg(f - F0, AHEAD);
            if (f < 16) {
                const int ks = f >> 2, kb = f & 3;
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) s[kb][qb] = Elem<T>::mfma16(fr[r], qf[qb][ks], s[kb][qb]);
            } else {
                const int j = (f - 16) >> 3, db = (f - 16) & 7;
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) o[db][qb] = Elem<T>::mfma16(fr[r], pf[j][qb], o[db][qb]);
                if (kSumOnMatrixPipe && db == 3) {
#pragma unroll
                    for (int qb = 0; qb < QB; ++qb) l_acc[qb] = Elem<T>::mfma16(ones, pf[j][qb], l_acc[qb]);
                }
            }
        };
        static_assert((F1 - F0) % 2 == 0 && AHEAD % 2 == 0, "fragments come in pairs");
#pragma unroll
        for (int f = F0; f < F1; f += 2) {
            __builtin_amdgcn_sched_barrier(0);
            use(f + 1);
            if (f + AHEAD < F1) fr[frag_reg(f + AHEAD - F0, AHEAD)] = read_frag(slot_c, slot, f + AHEAD);
            __builtin_amdgcn_sched_barrier(0);
            use(f);
            if (f + 1 + AHEAD < F1) fr[frag_reg(f + 1 + AHEAD - F0, AHEAD)] = read_frag(slot_c, slot, f + 1 + AHEAD);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I16 = std::integral_constant<int, 16>;
    using I32 = std::integral_constant<int, 32>;
    using Dyn = std::integral_constant<int, -1>;

    // softmax of tile `tile`. CSLOT >= 0: the four copies of the pair in ring slot CSLOT ride along, full tiles from the
    // running pointers; CSLOT == -1: general copies of pair cq; CSLOT == -2: none.
    auto softmax_tile = [&](float4v(&s)[4][QB], int tile, V8(&pf)[2][QB], auto cslot_c, int cq) {
        constexpr int CSLOT = decltype(cslot_c)::value;
        auto copy = [&](auto which_c) {
            constexpr int W = decltype(which_c)::value;   // 0, 1: halves of K; 2, 3: halves of V
            if constexpr (CSLOT >= 0) {
                if constexpr (W < 2) copy16_global_to_lds_at<CSLOT * TILE_BYTES + W * NWAVES * 1024>(k_next, k_lane_off[W], lds_wave);
                else copy16_global_to_lds_at<VBUF0 + CSLOT * TILE_BYTES + (W - 2) * NWAVES * 1024>(v_next, v_lane_off[W - 2], lds_wave);
            } else if constexpr (CSLOT == -1) {
                if constexpr (W < 2) issue_k1(cq, W);
                else issue_v1(cq, W - 2);
            }
        };
        const int key0 = tile * BN;
        const bool need_mask = (key0 + BN > kv_valid) || (causal && (key0 + BN - 1 > q_wave0 + shift));
        copy(std::integral_constant<int, 0>{});
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
        // necessarily its running maximum. A lane asks for it to move when one of ITS scores exceeds m_thr = m_run +
        // 2^kLazyLog2 / scale; then (any lane of the wave asked) the four lanes of every query agree on the tile's maximum
        // and the reference is raised to the running maximum. Otherwise P = exp2((S - m_run) c) <= 2^kLazyLog2 everywhere.
        // maximum of the 16 scores a lane holds of a query: two chains of v_max3 per query, the chains of both queries
        // interleaved (written in the order they are to run: between an instruction of an assembly statement and a
        // dependent one right behind it the compiler puts a wait state, an issue slot each)
        float mx[QB], mc[QB];
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) mx[qb] = max3v(s[0][qb][0], s[0][qb][1], s[0][qb][2]);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) mc[qb] = max3v(s[0][qb][3], s[1][qb][0], s[1][qb][1]);
#pragma unroll
        for (int kb = 1; kb < 4; ++kb) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) mx[qb] = max3v(mx[qb], s[kb][qb][2], s[kb][qb][3]);
            if (kb < 3) {
#pragma unroll
                for (int qb = 0; qb < QB; ++qb) mc[qb] = max3v(mc[qb], s[kb + 1][qb][0], s[kb + 1][qb][1]);
            }
        }
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) mx[qb] = max3v(mx[qb], mc[qb], mc[qb]);
        // the second copy sits between the max tree and the compare that reads its result: the compiler puts wait states
        // between an assembly statement and a dependent instruction, and these instructions take their place
        __builtin_amdgcn_sched_barrier(0);
        copy(std::integral_constant<int, 1>{});
        __builtin_amdgcn_sched_barrier(0);
        bool raise = false;
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) raise = raise || (mx[qb] > m_thr[qb]);
        if (__builtin_amdgcn_ballot_w64(raise) != 0) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb) {
                const float m_new = fmaxf(m_run[qb], quad_max(mx[qb]));
                const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                const float alpha = fast_exp2((m_run[qb] - m_use) * scale_log2);
                m_run[qb] = m_new;
                m_thr[qb] = m_new + lazy_margin;
                neg_ms[qb] = -m_use * scale_log2;
                // in place, as assembly: left to itself the compiler writes the products to other registers, and the common
                // path (no rescale) then pays for 72 register moves to meet it at the join
                l_acc[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < 8; ++db) o[db][qb] *= alpha;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int qb = 0; qb < QB; ++qb)
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                for (int e = 0; e < 4; ++e) s[kb][qb][e] = __builtin_fmaf(s[kb][qb][e], scale_log2, neg_ms[qb]);
        __builtin_amdgcn_sched_barrier(0);
        copy(std::integral_constant<int, 2>{});
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
            for (int qb = 0; qb < QB; ++qb)
#pragma unroll
                for (int e = 0; e < 4; ++e) s[kb][qb][e] = fast_exp2(s[kb][qb][e]);
            if (kb == 1) {
                __builtin_amdgcn_sched_barrier(0);
                copy(std::integral_constant<int, 3>{});
                __builtin_amdgcn_sched_barrier(0);
            }
        }
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
        if constexpr (CSLOT >= 0) {
            k_next += k_tile_bytes;
            v_next += v_tile_bytes;
        }
    };

    // ---- persistent loop over the work items of this workgroup ----------------------------------------------------------
    // The first pairs and the Q fragments of the NEXT item are requested as soon as the last barrier of the current one is
    // passed (every wave has finished reading LDS, and the Q registers are free), in front of the current item's epilogue:
    // normalising and storing O runs while those loads are on their way, and the workgroup never goes back to the
    // dispatcher between items.
    MI355_TL(unsigned long long tl_tiles = 0;)
    set_item(0);   // a launch has no more workgroups than items
    load_q();
    if (n_tiles > 0) issue_first_pairs();
    for (int round = 0;;) {
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            m_run[qb] = -INFINITY;
            m_thr[qb] = -INFINITY;
            neg_ms[qb] = 0.f;
            l_acc[qb] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int db = 0; db < 8; ++db) o[db][qb] = float4v{0.f, 0.f, 0.f, 0.f};
        }
        if (n_tiles > 0) {
            // pairs 0, 1, 2 and Q have landed (and the stores of the previous item's epilogue have been accepted)
            wait_vmcnt<0>();
            __syncthreads();
            if (late) end_phase();   // waves 4..7 idle during P0

            float4v s[4][QB];
            V8 pf[2][QB];
            V8 fr[AHEAD];
            MI355_TL(if (round == 0) tl_w[1] = timeline::wall_clock(); const unsigned long long tl_c0 = timeline::shader_cycles();)
            preload(I0{}, std::integral_constant<int, 0>{}, 0, fr);
            __builtin_amdgcn_s_setprio(1);
            mfma_phase(I0{}, I16{}, std::integral_constant<int, 0>{}, 0, s, pf, fr);               // S(0) alone
            __builtin_amdgcn_s_setprio(0);
            pin_s(s);
            end_phase();
            // tile step j: softmax(j) (with the copies of pair j + 3), then S(j+1) and O += V(j)^T P(j) on pair j + 1
            auto step = [&](auto u_c, int j) {
                constexpr int U = decltype(u_c)::value;   // j % NBUF in the unrolled loop, -1 in the general one
                using CopySlot = std::integral_constant<int, (U >= 0 ? (U + 3) % NBUF : -1)>;
                using ReadSlot = std::integral_constant<int, (U >= 0 ? (U + 1) % NBUF : -1)>;
                softmax_tile(s, j, pf, CopySlot{}, j + 3);
                pin_p(pf);
                preload(I0{}, ReadSlot{}, (j + 1) & (NBUF - 1), fr);
                end_phase();
                __builtin_amdgcn_s_setprio(1);
                mfma_phase(I0{}, I32{}, ReadSlot{}, (j + 1) & (NBUF - 1), s, pf, fr);
                __builtin_amdgcn_s_setprio(0);
                pin_s(s);
                pin_o();
                end_phase();
            };
            // unrolled loop: while the pair copied in step j (tiles j + 3 and j + 2) is made of full tiles
            const int j_fast = max(0, min(n_full - 3, n_tiles - 1)) & ~(NBUF - 1);
            int j = 0;
            for (; j < j_fast; j += NBUF) {
                step(std::integral_constant<int, 0>{}, j);
                step(std::integral_constant<int, 1>{}, j + 1);
                step(std::integral_constant<int, 2>{}, j + 2);
                step(std::integral_constant<int, 3>{}, j + 3);
            }
            for (; j + 1 < n_tiles; ++j) step(Dyn{}, j);
            softmax_tile(s, n_tiles - 1, pf, std::integral_constant<int, -2>{}, 0);
            pin_p(pf);
            preload(I16{}, Dyn{}, n_tiles & (NBUF - 1), fr);
            end_phase();
            mfma_phase(I16{}, I32{}, Dyn{}, n_tiles & (NBUF - 1), s, pf, fr);     // O += V(last)^T P(last) alone
            end_phase();
            if (!late) end_phase();  // waves 0..3 idle while waves 4..7 finish
            // behind this barrier no wave reads LDS any more; the copies past the end of the item that are still on their
            // way must land before the next item's pairs are sent into the same slots (or the workgroup ends)
            wait_vmcnt<0>();
            MI355_TL(tl_w[2] = timeline::wall_clock(); tl_c[1] += timeline::shader_cycles() - tl_c0; tl_tiles += (unsigned long long)n_tiles;)
        }

        // what the epilogue needs of the item just finished, then on to the next one
        T* const o_item = Oh;
        const int q_item0 = q_wave0;
        float* const lse_item = LSE == nullptr ? nullptr : LSE + ((long)b * Hq + hq) * (long)Sq;
        const bool more = set_item(++round);
        if (more) {
            load_q();
            if (n_tiles > 0) issue_first_pairs();
        }
        // ---- finalize: O / l, LSE: lane holds O[query 16 qb + c][d = 16 db + 4 g + 0..3] --------------------------------
#pragma unroll
        for (int qb = 0; qb < QB; ++qb) {
            const float l_tot = kSumOnMatrixPipe ? l_acc[qb][0] : quad_sum(l_acc[qb][0]);
            const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
            const int qi = q_item0 + qb * 16 + c16;
            if (qi < Sq) {
                T* orow = o_item + qi * o_row + 4 * g;
#pragma unroll
                for (int db = 0; db < 8; ++db) {
                    V4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = (T)(o[db][qb][e] * inv);
                    *(V4*)(orow + db * 16) = v;
                }
                if (lse_item != nullptr && g == 0)
                    lse_item[qi] = (l_tot > 0.f) ? (m_run[qb] * scale_log2 + __builtin_log2f(l_tot)) * 0.69314718055994531f : -INFINITY;
            }
        }
        if (!more) break;
    }
    MI355_TL(
        wait_vmcnt<0>();   // the stores of this wave have been accepted
        tl_w[3] = timeline::wall_clock();
        if (tid == 0 && blockIdx.x < timeline::kMaxWorkgroups) {
            unsigned long long* rec = fmha_fwd_stamps + (long)blockIdx.x * timeline::kSlots;
            rec[0] = tl_w[0]; rec[1] = tl_w[1]; rec[2] = tl_w[2]; rec[3] = tl_w[3];
            rec[4] = 0; rec[5] = tl_c[1]; rec[6] = tl_tiles; rec[7] = 0;
        })
}

// number of CUs of the current device (asked once per device)
static hipError_t compute_units(int& cus) {
    static std::atomic<int> cached[DynamicLdsOnce::kMaxDevices] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    const bool tracked = dev >= 0 && dev < DynamicLdsOnce::kMaxDevices;
    if (tracked && (cus = cached[dev].load(std::memory_order_relaxed)) > 0) return hipSuccess;
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev); e != hipSuccess) return e;
    if (cus < 1) return hipErrorInvalidDevice;
    if (tracked) cached[dev].store(cus, std::memory_order_relaxed);
    return hipSuccess;
}

template <typename T, int QB>
static hipError_t launch_fmha_pingpong(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq,
                                   int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd,
                                   hipStream_t stream) {
    constexpr int BM = 128 * QB;
    constexpr int LDS = 8 * fmha::TILE_BYTES;
    auto kern = fmha_fwd_pingpong_kernel<T, QB>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), LDS); e != hipSuccess) return e;
    const int q_tiles = (Sq + BM - 1) / BM;
    const long items = (long)q_tiles * Hq * B;
    if (items > 0x7fffffffL) return hipErrorInvalidValue;
    // one workgroup per CU at most (128 KiB of LDS each: a CU holds one); a multiple of 8 when the (batch, kv head) groups
    // divide over the 8 XCDs, so that fmha_work_item can give every XCD whole groups
    int cus = 0;
    if (hipError_t e = compute_units(cus); e != hipSuccess) return e;
    long blocks = items < cus ? items : cus;
    if (((long)Hkv * B) % 8 == 0 && blocks >= 8) blocks &= ~7L;
    const float scale_log2 = scale * 1.4426950408889634f;
    kern<<<dim3((unsigned)blocks), dim3(512), LDS, stream>>>(Q, K, V, O, LSE, B, Hq, Hkv, Sq, Sk, scale_log2, causal, kv_valid,
                                                             q_tiles, sd, 1, 0);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------------
// A few queries against a long cache (a chunk of a prompt appended to earlier chunks): one work item per (head, q tile)
// would leave most CUs idle behind a walk over all keys, so the keys are cut into ranges, every (range, head, q tile) is
// a work item of the same kernel (SEG) and a second kernel merges the ranges:
//   O = sum_s w_s O_s / sum_s w_s,  w_s = exp(LSE_s - max_s LSE_s),  LSE = max_s LSE_s + log(sum_s w_s)
// (a range without a visible key has LSE_s = -inf and weight 0; a row without any visible key gets O = 0, LSE = -inf).
// The partial results live in a workspace of the library's own, one buffer per (device, stream), allocated at first use
// and replaced by a larger one when a call needs more (never freed: a captured graph may hold its address). A call that
// cannot get it (its stream is being captured and has none yet) runs the kernel without ranges instead.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMaxSegments = 8;

template <typename T>
__global__ __launch_bounds__(256) void fmha_merge_segments_kernel(const T* __restrict__ Opart, const float* __restrict__ LSEpart,
                                                                  T* __restrict__ O, float* __restrict__ LSE, int B, int Hq, int Sq,
                                                                  int segments, FmhaStrides sd) {
    using V2 = typename Elem<T>::v2;
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);   // one wave per (batch, head, query)
    const long rows = (long)B * Hq * Sq;
    if (row >= rows) return;
    const int q = (int)(row % Sq);
    const long bh = row / Sq;
    const int h = (int)(bh % Hq), b = (int)(bh / Hq);
    // at most kMaxSegments ranges: every load of the row is issued before the first use
    float ls[kMaxSegments];
    V2 vs[kMaxSegments];
#pragma unroll
    for (int s = 0; s < kMaxSegments; ++s) {
        const int sc = s < segments ? s : 0;
        ls[s] = LSEpart[(long)sc * rows + row];
        vs[s] = *(const V2*)(Opart + ((long)sc * rows + row) * fmha::D + 2 * lane);
        if (s >= segments) ls[s] = -INFINITY;
    }
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < kMaxSegments; ++s) m = fmaxf(m, ls[s]);
    float acc0 = 0.f, acc1 = 0.f, denom = 0.f;
    if (m > -INFINITY) {
#pragma unroll
        for (int s = 0; s < kMaxSegments; ++s) {
            const float w = __expf(ls[s] - m);   // exp(-inf) = 0: a range without a visible key, or beyond `segments`
            acc0 += w * (float)vs[s][0];
            acc1 += w * (float)vs[s][1];
            denom += w;
        }
    }
    const float inv = denom > 0.f ? 1.f / denom : 0.f;
    V2 out;
    out[0] = (T)(acc0 * inv);
    out[1] = (T)(acc1 * inv);
    *(V2*)(O + b * sd.o_batch + h * sd.o_head + q * sd.o_row + 2 * lane) = out;
    if (LSE != nullptr && lane == 0) LSE[row] = denom > 0.f ? m + __logf(denom) : -INFINITY;
}

static hipError_t segment_workspace(size_t bytes, hipStream_t stream, char** out) {
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
        const size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes + bytes / 2;
        void* fresh = nullptr;
        e = hipMalloc(&fresh, want);
        if (e != hipSuccess) return e;
        b.ptr = fresh;   // the previous buffer, if any, stays allocated (see above)
        b.size = want;
    }
    *out = static_cast<char*>(b.ptr);
    return hipSuccess;
}

// How a call cuts its keys: `segments` ranges (0: not cut) walked by work items of 128 `qb` queries.
// 128-query items: at most 128 of them; about one item per CU, at least 1024 keys per range (2048 where only two ranges
// fit), at most 8 ranges. Measured, 32/8 heads, causal, one walk / ranges (us): 64 queries over 8192 keys 90 / 25, 128 over
// 8192 92 / 28, 256 over 8192 92 / 44, 128 over 32768 343 / 75, 2 x 128 over 4096 50 / 29, 4 x 128 over 8192 94 / 79; two
// ranges of 1024 keys lose (512 over 2048: 29 / 33).
// 256-query items (every K / V fragment feeds two MFMAs) where they fill the machine with ranges of at least 2048 keys: at
// most 128 items, at least 192 (item, range) pairs, at most an eighth of the q tiles empty. Measured, 128- / 256-query
// items over ranges (us): 512 over 8192 81 / 69, 768 over 8192 105 (one walk) / 102, 1024 over 8192 127 (one walk) / 124,
// 256 over 32768 138 / 120, 512 over 32768 262 / 220, 1024 over 32768 493 (one walk) / 423, 2 x 256 over 8192 78 / 71,
// 64/8 heads 256 over 16384 139 / 120; but 256 over 8192 (8 ranges of 1024 keys) 44 / 45, 384 over 8192 65 / 67.
struct KeyRangePlan {
    int segments = 0;
    int qb = 1;
};

static KeyRangePlan key_range_plan(int B, int Hq, int Sq, int kv_valid) {
    KeyRangePlan plan;
    if (kv_valid < 2048) return plan;
    const long q256 = (Sq + 255) / 256, items256 = q256 * Hq * B;
    if (Sq >= 256 && q256 * 256 - Sq <= Sq / 8 && items256 <= 128) {
        long s = 256 / items256;
        if (s > kMaxSegments) s = kMaxSegments;
        if (s > kv_valid / 2048) s = kv_valid / 2048;
        if (s >= 2 && items256 * s >= 192) {
            plan.segments = (int)s;
            plan.qb = 2;
            return plan;
        }
    }
    const long items = (long)((Sq + 127) / 128) * Hq * B;
    if (items > 128) return plan;
    long s = 256 / items;
    if (s > kMaxSegments) s = kMaxSegments;
    if (s > kv_valid / 1024) s = kv_valid / 1024;
    if (s == 2 && kv_valid < 4096) return plan;
    if (s >= 2) plan.segments = (int)s;
    return plan;
}

size_t fmha_key_range_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    if (fmha_decode_applicable(B, Hq, Hkv, Sq, Sk, kv_valid_len)) return 0;
    const KeyRangePlan plan = key_range_plan(B, Hq, Sq, kv_valid_len);
    return (size_t)plan.segments * B * Hq * Sq * (fmha::D * 2 + sizeof(float));   // fp16 / bf16 partial outputs, fp32 LSE
}

size_t fmha_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    const size_t decode = fmha_decode_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len);
    return decode > 0 ? decode : fmha_key_range_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len);
}

template <typename T, int QB>
static hipError_t launch_fmha_segmented(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq, int Hkv, int Sq,
                                        int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd, int segments,
                                        char* caller_ws, hipStream_t stream) {
    constexpr int LDS = 8 * fmha::TILE_BYTES;
    auto kern = fmha_fwd_pingpong_kernel<T, QB, true>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), LDS); e != hipSuccess) return e;
    const int seg_len = ((kv_valid + segments - 1) / segments + 63) & ~63;
    const long rows = (long)B * Hq * Sq;
    const size_t o_bytes = (size_t)segments * rows * fmha::D * sizeof(T);
    const size_t bytes = o_bytes + (size_t)segments * rows * sizeof(float);
    char* ws = caller_ws;   // memory of the caller (large enough: see fmha_fwd_dispatch), or the library's own
    if (ws == nullptr)
        if (hipError_t e = segment_workspace(bytes, stream, &ws); e != hipSuccess) return e;
    T* o_part = reinterpret_cast<T*>(ws);
    float* lse_part = reinterpret_cast<float*>(ws + o_bytes);
    const int q_tiles = (Sq + 128 * QB - 1) / (128 * QB);
    const long items = (long)q_tiles * Hq * B * segments;
    int cus = 0;
    if (hipError_t e = compute_units(cus); e != hipSuccess) return e;
    long blocks = items < cus ? items : cus;
    if (((long)Hkv * B * segments) % 8 == 0 && blocks >= 8) blocks &= ~7L;
    const float scale_log2 = scale * 1.4426950408889634f;
    kern<<<dim3((unsigned)blocks), dim3(512), LDS, stream>>>(Q, K, V, o_part, lse_part, B, Hq, Hkv, Sq, Sk, scale_log2, causal, kv_valid,
                                                             q_tiles, sd, segments, seg_len);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    fmha_merge_segments_kernel<T><<<dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, stream>>>(o_part, lse_part, O, LSE, B, Hq, Sq, segments, sd);
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
    const size_t range_bytes = (variant == 0 || variant == 3) ? fmha_key_range_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len) : 0;
    const bool caller_ws = ws.kind == FmhaWorkspace::kCaller && ws.ptr != nullptr && ws.bytes >= range_bytes &&
                           reinterpret_cast<uintptr_t>(ws.ptr) % 16 == 0;
    if (range_bytes > 0 && (ws.kind == FmhaWorkspace::kLibrary || caller_ws)) {
        const KeyRangePlan plan = key_range_plan(B, Hq, Sq, kv_valid_len);
        char* const mem = caller_ws ? static_cast<char*>(ws.ptr) : nullptr;
        const hipError_t e =
            plan.qb == 2 ? launch_fmha_segmented<T, 2>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, plan.segments, mem, stream)
                         : launch_fmha_segmented<T, 1>(q, k, v, o, LSE, B, Hq, Hkv, Sq, Sk, scale, causal, kv_valid_len, sd, plan.segments, mem, stream);
        // without the workspace (none yet on a stream that is being captured, or no memory) the keys are walked in one go
        if (variant == 3 || (e != hipErrorStreamCaptureUnsupported && e != hipErrorOutOfMemory)) return e;
        (void)hipGetLastError();
    }
    if (variant == 3) return hipErrorInvalidConfiguration;   // the test hook asked for key ranges where they do not apply
    if (variant == 0) {
        // 256-query workgroups (every K / V fragment feeds two MFMAs) once their work items fill the machine: clearly more
        // of them than CUs for a causal problem (with about one per CU it runs as long as its heaviest item, and 128-query
        // items balance better), one per CU otherwise. Measured (b x heads q/kv x s, 128- / 256-query items, us): causal
        // 1 x 32/8 x 1024 20 / 30, 1 x 32/8 x 2048 45 / 51, 2 x 32/8 x 1024 30 / 32, 1 x 16/16 x 4096 76 / 88,
        // 1 x 8/8 x 8192 139 / 163, 2 x 8/2 x 4096 76 / 88, but 32 x 32/8 x 256 68 / 64, 8 x 32/8 x 512 42 / 39,
        // 1 x 32/8 x 3000 92 / 78, 2 x 32/8 x 1536 56 / 50, 4 x 32/8 x 1024 57 / 50, 1 x 32/8 x 4096 149 / 126,
        // 16 x 32/8 x 768 148 / 128, 4 x 32/8 x 2048 170 / 147; not causal 2 x 32/8 x 1024 42 / 36, 1 x 32/8 x 2048 73 / 62,
        // 4 x 32/32 x 1024 89 / 71. A problem that is not causal and has a few more 256-query items than CUs runs as long
        // as two of them, on a quarter of the machine at the end; twice as many 128-query items are three to a CU then,
        // each a little more than half as long (1 x H/1 x 2048 with H = 33 .. 44, i.e. 264 .. 352 items: 94.5 - 97.6 us
        // against 99.9; 368 items 99.6 / 100.0; 384 items 102.6 / 100.1).
        // (A causal problem whose queries are the last of at least twice as many keys - a chunk of new tokens against a
        // cache - has items of nearly equal length, like a problem that is not causal: 1 x 32/8 x 2048 queries over 8192
        // keys 223 / 200.)
        const long wg256 = (long)((Sq + 255) / 256) * Hq * B;
        const bool uneven = causal && Sk < 2 * (long)Sq;
        variant = (Sq >= 256 && wg256 >= (uneven ? 320 : 256)) ? 2 : 1;
        if (!causal && wg256 > 256 && wg256 <= 352) variant = 1;
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
