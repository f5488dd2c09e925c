// Decode-shaped attention forward for gfx950 (MI355X): few query rows per kv head, long key sequence.
//
// The reference runs its generation step (`is_decode`, one query row padded to 64 by ops.py:19-25) through the
// prefill kernel, one workgroup per (batch, q head) walking all keys (semi/fmha_2_amd.cpp:341-356); that leaves
// almost the whole GPU idle and is bound by one workgroup's memory rate. Here the step is a split-KV
// ("flash-decoding") pass in ONE launch, HBM-bound by the single read of K and V:
//
//   * a workgroup = (batch, kv head, key range); about one workgroup per CU. The query rows of all q heads that share
//     the kv head are packed side by side as the (up to 32) columns of the S^T = K Q^T product, so K and V are read once
//     per kv head, not once per q head.
//   * the waves of a workgroup cut its key range into contiguous pieces; each wave streams its piece in tiles of 32 keys
//     through a private LDS pipeline (direct-to-LDS copies, no workgroup barriers while streaming) and runs the
//     register-resident online softmax of the prefill kernel.
//   * the waves' results are combined through LDS and written as one unnormalised partial result per workgroup
//     (O~ [128], m, l per column, fp32) to a workspace; the workgroup then takes a ticket from a counter of its
//     (batch, kv head), and the one that draws the last ticket combines all partials of that pair,
//     O = sum_s 2^((m_s - m) c) O~_s / sum_s 2^((m_s - m) c) l_s, writes O and LSE and puts the counter back to zero.
//     With a single key range per (batch, kv head) the workgroup writes O and LSE directly and touches no workspace.
//
// Mask semantics are those of the prefill kernel (keys >= kv_valid_len masked; causal: key j visible to query i
// iff j <= i + Sk - Sq).
#include <atomic>
#include <map>
#include <mutex>
#include <utility>

#include "mi355_common.h"
#include "mi355_serving_internal.h"
#include "mi355_timeline.h"

namespace mi355 {

// profiling build: per workgroup, wall clock at [entry, first tile landed, key range done, partial results stored, ticket
// drawn, merge: partial results landed, merge: summed, exit] (0 = the workgroup did not get there)
MI355_TL(static __device__ unsigned long long fmha_decode_stamps[timeline::kMaxWorkgroups * timeline::kSlots];)

namespace dec {
constexpr int D = 128;
constexpr int TK = 32;                       // keys per tile
constexpr int ROW_BYTES = D * 2;             // 256
constexpr int TILE_BYTES = TK * ROW_BYTES;   // 8 KiB
constexpr int STAGE_BYTES = 2 * TILE_BYTES;  // K + V
constexpr float kLazyLog2 = 8.f;             // rescale only when a column maximum grows by more than 2^8
constexpr int COPIES = 2 * (TILE_BYTES / 1024);  // 16 copy instructions per stage
constexpr int PART_STRIDE = D + 4;           // floats per (workgroup, column): O~[128], m, l, 2 pad (keeps rows 16-byte aligned)
// Ticket counters lie this many 32-bit words (256 bytes) apart. Device-scope atomics of workgroups on different XCDs are
// carried out at the memory side, one after the other per address range: with the counters of all (batch, kv head)
// pairs in one 64-byte line, the 256 tickets of a call queued up behind each other (~12 ns each, 3 us from the first to
// the last at batch 1); 256 bytes apart they proceed side by side (a larger stride brought nothing more).
constexpr int kCounterStride = 64;
// The counters occupy a region of FIXED size at the start of every workspace, whatever the call: a workspace is shared by
// calls of different shapes, each of which leaves its counters at zero, and a region that grew and shrank with the number
// of (batch, kv head) pairs would let one call's partial results land where the next call keeps its counters. A call is
// cut into several key ranges only while it has at most kMaxSplitPairs pairs.
constexpr int kMaxSplitPairs = 255;
constexpr size_t kCounterBytes = size_t(kMaxSplitPairs + 1) * kCounterStride * sizeof(unsigned);   // 64 KiB

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

// Workgroup wg = (b * Hkv + hkv) * splits + s covers key tiles [s * tiles_per_split, (s + 1) * tiles_per_split).
// WAVES waves with NSTAGE pipeline stages of 16 KiB each. <4, 2> (one wave per SIMD, one tile in flight behind the one
// being consumed, 128 KiB of LDS) measured better than <3, 3> for short and for long key ranges alike.
template <typename T, int WAVES, int NSTAGE>
__global__ __launch_bounds__(WAVES * 64) void fmha_decode_kernel(
    const T* __restrict__ Q, const T* __restrict__ K, const T* __restrict__ V, T* __restrict__ O, float* __restrict__ LSE,
    float* part, unsigned* counters, int B, int Hq, int Hkv, int Sq, int Sk, float scale_log2, int causal, int kv_valid,
    int splits, int tiles_per_split, FmhaStrides sd) {
    using namespace dec;
    using V8 = typename Elem<T>::v8;
    MI355_TL(unsigned long long tl[8] = {timeline::wall_clock(), 0, 0, 0, 0, 0, 0, 0};
             auto tl_dump = [&]() {
                 if (threadIdx.x == 0 && blockIdx.x < timeline::kMaxWorkgroups)
                     for (int i = 0; i < 8; ++i) fmha_decode_stamps[(long)blockIdx.x * timeline::kSlots + i] = tl[i];
             };)
    constexpr int WAVE_BYTES = NSTAGE * STAGE_BYTES;
    constexpr int NTHREADS = WAVES * 64;
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    MI355_LDS char* wbase = (MI355_LDS char*)smem_raw + wave * WAVE_BYTES;

    const int h = lane >> 5;
    const int l32 = lane & 31;
    const int s_idx = blockIdx.x % splits;
    const int bh = blockIdx.x / splits;
    const int hkv = bh % Hkv;
    const int b = bh / Hkv;
    const int group = Hq / Hkv;
    const int ncols = group * Sq;  // <= 32
    const int shift = Sk - Sq;

    const T* Kh = K + b * sd.k_batch + hkv * sd.k_head;
    const T* Vh = V + b * sd.v_batch + hkv * sd.v_head;

    // this workgroup's tiles, and this wave's contiguous piece of them (possibly empty)
    const int tiles = (kv_valid + TK - 1) / TK;
    const int g_begin = s_idx * tiles_per_split;
    const int g_end = min(g_begin + tiles_per_split, tiles);
    const int per_wave = (max(g_end - g_begin, 0) + WAVES - 1) / WAVES;
    const int t_begin = min(g_begin + wave * per_wave, g_end);
    const int t_end = min(t_begin + per_wave, g_end);

    // copy i (0..7) of a tile covers rows 4i + lane/16, chunk position lane%16; addresses = wave-uniform tile base (scalar
    // registers) + 32-bit lane offset; rows past the last valid key are clamped onto it (masked later, but V must not
    // feed NaNs into 0 * V)
    const int c_row = lane >> 4;
    const uint32_t k_row_bytes = (uint32_t)sd.k_row * 2, v_row_bytes = (uint32_t)sd.v_row * 2;
    const uint32_t kcol = (lane & 15);
    auto issue_stage = [&](int tile, int slot) {
        MI355_LDS char* st = wbase + slot * STAGE_BYTES;
        const int tile_u = __builtin_amdgcn_readfirstlane(tile);
        const char* kb = (const char*)Kh + (long)tile_u * TK * sd.k_row * 2;
        const char* vb = (const char*)Vh + (long)tile_u * TK * sd.v_row * 2;
        const int last = kv_valid - 1 - tile_u * TK;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int row = 4 * i + c_row;
            copy16_global_to_lds(kb, (uint32_t)min(row, last) * k_row_bytes + ((kcol ^ swz_k(row)) << 4), st + i * 1024);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            int row = 4 * i + c_row;
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
    // each wave starts at a different tile of its piece and wraps around (the online softmax does not care about the
    // order): waves whose pieces lie a large power of two apart then do not walk the same memory channels in step
    const int rot = n_loc > 0 ? ((blockIdx.x * WAVES + wave) * 5) % n_loc : 0;
    auto tile_of = [&](int i) { int r = i + rot; return t_begin + (r >= n_loc ? r - n_loc : r); };
    int issued = t_begin;
#pragma unroll
    for (int i = 0; i < NSTAGE - 1; ++i)
        if (issued < t_end) {
            issue_stage(tile_of(issued - t_begin), i);
            ++issued;
        }
    // Everything about the queries comes behind the first key / value copies, so that those leave as early as possible
    // and the latency of the query fetch hides under theirs.
    // column c of the packed query block = (q head hkv*group + c / Sq, query row c % Sq)
    const int col = min(l32, ncols - 1);
    const int hq = hkv * group + col / Sq;
    const int qi = col % Sq;
    const T* qp = Q + b * sd.q_batch + hq * sd.q_head + qi * sd.q_row + 8 * h;
    const int lim = causal ? min(kv_valid - 1, qi + shift) : kv_valid - 1;  // last visible key of this column
    // smallest such limit over the wave: tiles that end at or before it need no mask code
    int lim_min = lim;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) lim_min = min(lim_min, __shfl_xor(lim_min, off, 64));
    lim_min = __builtin_amdgcn_readfirstlane(lim_min);
    V8 qf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) qf[ks] = *(const V8*)(qp + ks * 16);
    // A use of the query fragments in front of the loop: the compiler waits for their loads where they are first used,
    // and it does not count the tile copies (inline assembly) among the loads in flight. With the first use inside the
    // loop that wait, "everything I know of has landed", came back on every iteration as vmcnt(0) in front of the S^T
    // products and held each tile's arithmetic until the NEXT tile's copies had landed too: no copy ever overlapped
    // arithmetic. Out here it waits once, for the first tile and the queries, which the first iteration needs anyway.
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) asm volatile("" : "+v"(qf[ks]));
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
        MI355_TL(if (tt0 == t_begin) tl[1] = timeline::wall_clock();)
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

    // ---- combine the waves of the workgroup through LDS (the pipelines are drained: their memory is free) ------------
    // per wave: O~ [ncols][128] floats, then m [32], l [32]
    const float l_tot = l_run + other_half(l_run);
    MI355_TL(tl[2] = timeline::wall_clock();)
    __syncthreads();
    MI355_LDS float* cmb = (MI355_LDS float*)smem_raw;
    const int wave_floats = ncols * D + 64;
    {
        MI355_LDS float* mine = cmb + wave * wave_floats;
        if (l32 < ncols) {
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    float4v v;
#pragma unroll
                    for (int q = 0; q < 4; ++q) v[q] = o[db][4 * p + q];
                    *(MI355_LDS float4v*)(mine + l32 * D + db * 32 + 8 * p + 4 * h) = v;
                }
            if (h == 0) {
                mine[ncols * D + l32] = m_run;
                mine[ncols * D + 32 + l32] = l_tot;
            }
        }
    }
    __syncthreads();
    const long row0 = ((long)b * Hq + (long)hkv * group) * Sq;   // LSE index of column 0 (columns are consecutive rows)
    // element idx = (column, d) of the workgroup's result; weights 2^((m_w - m) c), 0 for waves without a visible key
    auto combined = [&](int c, int d, float& m_out, float& l_out) {
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) m = fmaxf(m, cmb[w * wave_floats + ncols * D + c]);
        float acc = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float mw = cmb[w * wave_floats + ncols * D + c];
            const float wgt = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((mw - m) * scale_log2);
            acc += wgt * cmb[w * wave_floats + c * D + d];
            l += wgt * cmb[w * wave_floats + ncols * D + 32 + c];
        }
        m_out = m;
        l_out = l;
        return acc;
    };
    if (splits == 1) {   // the only key range of this (batch, kv head): the result is final
        for (int idx = tid; idx < ncols * D; idx += NTHREADS) {
            const int c = idx >> 7, d = idx & (D - 1);
            float m, l;
            const float acc = combined(c, d, m, l);
            const int chq = hkv * group + c / Sq, cqi = c % Sq;
            O[b * sd.o_batch + chq * sd.o_head + cqi * sd.o_row + d] = (T)((l > 0.f) ? acc / l : 0.f);
            if (LSE != nullptr && d == 0)
                LSE[row0 + c] = (l > 0.f) ? (m * scale_log2 + __builtin_log2f(l)) * 0.69314718055994531f : -INFINITY;
        }
        MI355_TL(wait_vmcnt<0>(); tl[7] = timeline::wall_clock(); tl_dump();)
        return;
    }
    // Partial results cross XCDs (each has its own L2). The hand-over from the workgroups that write them to the one that
    // merges them is ordered by instructions, not by a release / acquire pair: a device-scope fence writes back and
    // invalidates a whole L2 here, and an acquire-release ticket costs 2.5-3 us per launch (b = 1 over 8192 keys: 13.8 us
    // against 11.0). What takes the fence's place, step by step:
    //   1. every partial result is stored with a device-scope atomic store, i.e. `global_store_dword .. sc1`: written through
    //      the XCD's L2 to memory, nothing of it stays dirty in a cache;
    //   2. `s_waitcnt vmcnt(0)` behind the stores: on gfx9-family parts a store leaves vmcnt only when the memory system has
    //      acknowledged it at the scope it was issued with. The wait is an assembly statement with a memory clobber, so the
    //      compiler keeps the stores in front of it;
    //   3. the workgroup barrier: all threads have passed their wait before thread 0 draws the ticket;
    //   4. the ticket is a device-scope atomic add, carried out at the memory side: the tickets of one counter are totally
    //      ordered, and the workgroup that draws the last one knows that every other workgroup of its (batch, kv head) has
    //      passed step 2;
    //   5. the merging workgroup reads the partial results with `global_load_dword[x4] .. sc1` (device-coherent: served from
    //      memory, not from a line its XCD's L2 may still hold from an earlier launch), issued behind the branch on the
    //      ticket's value, which the hardware cannot pass before the atomic has returned.
    // tests/test_inline_asm_loads_cpu.py checks 1, 2 and 5 in the generated code.
    float* mypart = part + (long)blockIdx.x * ncols * PART_STRIDE;
    for (int idx = tid; idx < ncols * D; idx += NTHREADS) {
        const int c = idx >> 7, d = idx & (D - 1);
        float m, l;
        __hip_atomic_store(mypart + c * PART_STRIDE + d, combined(c, d, m, l), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d == 0) {
            __hip_atomic_store(mypart + c * PART_STRIDE + D, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(mypart + c * PART_STRIDE + D + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // ---- ticket: the workgroup that completes the set of key ranges of (b, hkv) merges them ----------------------------
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this thread's partial results have reached memory before the ticket is drawn
    MI355_TL(tl[3] = timeline::wall_clock();)
    __syncthreads();
    MI355_LDS unsigned* ticket_sh = (MI355_LDS unsigned*)(cmb + WAVES * wave_floats);
    if (tid == 0) *ticket_sh = __hip_atomic_fetch_add(&counters[(long)bh * kCounterStride], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    MI355_TL(tl[4] = timeline::wall_clock();)
    if (*ticket_sh != (unsigned)(splits - 1)) {
        MI355_TL(tl[7] = tl[4]; tl_dump();)
        return;
    }
    // last ticket: every other workgroup of (b, hkv) drew its ticket after its partial results had reached memory.
    // They are read back with device-coherent loads (sc1), many in flight per thread: one memory round trip for the
    // statistics, then one per 16 key ranges for the outputs.
    const float* base = part + (long)bh * splits * ncols * PART_STRIDE;
    const long split_stride = (long)ncols * PART_STRIDE;
    MI355_LDS float* st_m = cmb;                          // [splits][ncols]: m_s
    MI355_LDS float* st_l = cmb + splits * ncols;         // [splits][ncols]: l_s
    constexpr int BATCH = 32;
    // BATCH loads of 16 bytes each: the outputs of key ranges sp0 .. sp0 + BATCH - 1 for 4 d of one column
    // (in groups of 8 key ranges, a group only when it holds a key range that exists: a call with 4 key ranges issues 8
    // loads per thread, not 32; within a group, key ranges past the last one repeat it and get weight zero)
    auto load_batch = [&](float4v(&v)[BATCH], const float* pc, int sp0) {
#pragma unroll
        for (int g8 = 0; g8 < BATCH; g8 += 8) {
            if (sp0 + g8 < splits) {
#pragma unroll
                for (int u = g8; u < g8 + 8; ++u) {
                    const float* pa = pc + (long)min(sp0 + u, splits - 1) * split_stride;
                    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[u]) : "v"(pa) : "memory");
                }
            }
        }
    };
    auto wait_batch = [](float4v(&v)[BATCH]) {   // the loads above have landed; nothing that uses v moves in front of this
        asm volatile("s_waitcnt vmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                       "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15])
                     :: "memory");
        asm volatile("" : "+v"(v[16]), "+v"(v[17]), "+v"(v[18]), "+v"(v[19]), "+v"(v[20]), "+v"(v[21]), "+v"(v[22]), "+v"(v[23]),
                          "+v"(v[24]), "+v"(v[25]), "+v"(v[26]), "+v"(v[27]), "+v"(v[28]), "+v"(v[29]), "+v"(v[30]), "+v"(v[31]));
    };
    // the first batch of this thread's first output element goes out before the statistics are fetched: one memory
    // round trip serves both
    float4v v[BATCH];
    const int n_out = ncols * (D / 4);   // output elements f = (column, group of 4 d)
    if (tid < n_out) load_batch(v, base + (tid >> 5) * PART_STRIDE + (tid & 31) * 4, 0);
    for (int i = tid; i < splits * ncols; i += NTHREADS) {
        const float* ps = base + (long)(i / ncols) * split_stride + (i % ncols) * PART_STRIDE + D;
        float ms, ls;
        asm volatile("global_load_dword %0, %2, off sc1\n\tglobal_load_dword %1, %2, off offset:4 sc1\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(ms), "=&v"(ls) : "v"(ps) : "memory");
        st_m[i] = ms;
        st_l[i] = ls;
    }
    MI355_TL(tl[5] = timeline::wall_clock();)
    __syncthreads();
    // The weight of key range s for column c, 2^((m_s - m_c) scale), is worked out once, by thread s * ncols + c, and left in
    // LDS together with its share of the row sum; the accumulation loop below then is two LDS reads and four
    // multiply-adds per key range.
    MI355_LDS float* st_w = cmb + 2 * splits * ncols;     // [splits][ncols]: weight of key range s
    MI355_LDS float* st_mc = cmb + 3 * splits * ncols;    // [ncols]: m_c
    for (int i = tid; i < splits * ncols; i += NTHREADS) {
        const int c = i % ncols;
        float m = -INFINITY;
        for (int sp0 = 0; sp0 < splits; sp0 += 8) {   // 8 independent LDS reads at a time
            float ms[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) ms[u] = st_m[min(sp0 + u, splits - 1) * ncols + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) m = fmaxf(m, ms[u]);
        }
        const float w = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((st_m[i] - m) * scale_log2);
        st_w[i] = w;
        st_l[i] *= w;
        if (i < ncols) st_mc[c] = m;
    }
    __syncthreads();
    for (int f = tid; f < n_out; f += NTHREADS) {
        const int c = f >> 5, d = (f & 31) * 4;
        const float* pc = base + c * PART_STRIDE + d;
        float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
        float l = 0.f;
        for (int sp0 = 0; sp0 < splits; sp0 += BATCH) {
            if (f != tid || sp0 != 0) load_batch(v, pc, sp0);
            // the weights of this batch, while its loads are in flight (all LDS reads first, so they overlap each other);
            // key ranges past the last one repeat it with weight zero
            float wgt[BATCH], ls[BATCH];
#pragma unroll
            for (int g8 = 0; g8 < BATCH; g8 += 8) {
                if (sp0 + g8 < splits) {
#pragma unroll
                    for (int u = g8; u < g8 + 8; ++u) {
                        const int sp = min(sp0 + u, splits - 1);
                        wgt[u] = st_w[sp * ncols + c];
                        ls[u] = st_l[sp * ncols + c];
                    }
#pragma unroll
                    for (int u = g8; u < g8 + 8; ++u) {
                        if (sp0 + u >= splits) wgt[u] = ls[u] = 0.f;
                        l += ls[u];
                    }
                }
            }
            wait_batch(v);
#pragma unroll
            for (int g8 = 0; g8 < BATCH; g8 += 8) {
                if (sp0 + g8 < splits) {
#pragma unroll
                    for (int u = g8; u < g8 + 8; ++u)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[e] += wgt[u] * v[u][e];
                }
            }
        }
        MI355_TL(tl[6] = timeline::wall_clock();)
        const float inv = (l > 0.f) ? 1.f / l : 0.f;
        const int chq = hkv * group + c / Sq, cqi = c % Sq;
        typename Elem<T>::v4 ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) ov[e] = (T)(acc[e] * inv);
        *(typename Elem<T>::v4*)(O + b * sd.o_batch + chq * sd.o_head + cqi * sd.o_row + d) = ov;
        if (LSE != nullptr && d == 0)
            LSE[row0 + c] = (l > 0.f) ? (st_mc[c] * scale_log2 + __builtin_log2f(l)) * 0.69314718055994531f : -INFINITY;
    }
    // ready for the next call that uses this workspace (a device-scope store like the tickets, which are the only other
    // accesses to the counter; the next launch on the stream starts after this one has ended)
    if (tid == 0) __hip_atomic_store(&counters[(long)bh * kCounterStride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    MI355_TL(wait_vmcnt<0>(); tl[7] = timeline::wall_clock(); tl_dump();)
}

// Sets the counters of a workspace whose contents are unknown (a caller's) to zero.
__global__ void fmha_decode_clear_kernel(unsigned* counters, int n) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) counters[i] = 0u;
}

bool fmha_decode_applicable(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    const int group = Hq / Hkv;
    return (long)group * Sq <= 32 && kv_valid_len >= 512 && Sk >= kv_valid_len && B >= 1;
}

namespace dec {
constexpr int kMaxSplits = 256;   // key ranges per (batch, kv head)
}   // up to this many tiles per wave: <4 waves, 2 stages>

// How a call is cut into workgroups, and what its workspace holds: one counter per (batch, kv head), kCounterStride
// words apart, then the partial results [workgroup][column][PART_STRIDE].
struct DecodePlan {
    int splits, tiles_per_split;
    long workgroups;
    size_t counter_bytes, bytes;   // bytes == 0: a single key range per (batch, kv head), no workspace
};
static DecodePlan decode_plan(int B, int Hq, int Hkv, int Sq, int kv_valid) {
    using namespace dec;
    const int ncols = (Hq / Hkv) * Sq;
    const int tiles = (kv_valid + TK - 1) / TK;
    const long pairs = (long)B * Hkv;
    // about one workgroup per CU; a key range is at least 8 tiles (two per wave)
    long splits = (256 + pairs / 2) / pairs;
    splits = (splits < 1 || pairs > kMaxSplitPairs) ? 1 : splits;
    const long max_splits = (tiles + 7) / 8;
    if (splits > max_splits) splits = max_splits;
    if (splits > kMaxSplits) splits = kMaxSplits;
    DecodePlan p;
    p.tiles_per_split = (int)((tiles + splits - 1) / splits);
    p.splits = (tiles + p.tiles_per_split - 1) / p.tiles_per_split;
    p.workgroups = pairs * p.splits;
    p.counter_bytes = p.splits > 1 ? kCounterBytes : 0;
    p.bytes = p.splits > 1 ? p.counter_bytes + (size_t)p.workgroups * ncols * PART_STRIDE * sizeof(float) : 0;
    return p;
}

size_t fmha_decode_workspace_bytes(int B, int Hq, int Hkv, int Sq, int Sk, int kv_valid_len) {
    if (!fmha_decode_applicable(B, Hq, Hkv, Sq, Sk, kv_valid_len)) return 0;
    return decode_plan(B, Hq, Hkv, Sq, kv_valid_len).bytes;
}

// The library's own workspace: one buffer per (device, stream), allocated on first use and replaced by a larger one when
// a call needs more. A buffer that has been handed to a kernel is NEVER freed: a HIP graph captured earlier may hold
// its address, so replaced buffers stay allocated until the process ends (each replacement is at least 1.5x larger, so
// together they hold less than three times the largest request), and so does the buffer of every stream that ever made
// such a call (at least 4 MiB each: a process that creates streams without end should hand in its own workspace,
// mi355_fmha_fwd_ws). Calls on one stream are ordered, so they can share a buffer; calls on different streams get
// different ones. Nothing can be allocated while the stream is capturing: such a call fails with
// hipErrorStreamCaptureUnsupported unless an earlier call on the same stream already made the buffer large enough (run
// the step once before capturing it, or hand in a workspace of your own). Only the calling stream's capture state can be
// seen from here: while ANOTHER stream of the process captures in global capture mode, a first or growing call (a
// hipMalloc) would invalidate that capture, so make those calls before any capture starts. `fresh_counters` tells the
// caller that the buffer is new and its ticket counters still have to be set to zero (on the calling stream, in front of
// the kernel: no synchronous fill of the whole buffer on the null stream).
static hipError_t decode_workspace(size_t bytes, hipStream_t stream, char** out, bool* fresh_counters) {
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
    *fresh_counters = false;
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
        *fresh_counters = true;
    }
    *out = static_cast<char*>(b.ptr);
    return hipSuccess;
}

// Static scratch for callers that must not allocate (mi355_fmha_fwd_noalloc): a fixed array in device memory, one copy
// per GPU the library is loaded on, held until the process ends; it starts out zeroed (so do its ticket counters). Host
// code never uses the symbol's name as an address: the device address is looked up once per device with
// hipGetSymbolAddress and kept. Every call on a GPU shares that GPU's array and relies on finding its ticket counters at
// zero, where every completed call leaves them: calls that overlap on one GPU race, and a call that does not run to its end
// (a kernel that is aborted, overlapping calls) leaves a counter that is not zero. From then on no workgroup of that
// (batch, kv head) draws the last ticket, O and LSE of its rows are not written and no error is reported, until the
// process ends; mi355_fmha_fwd_ws (counters zeroed on every call) is the entry point that does not depend on history.
constexpr size_t kStaticScratchBytes = size_t(4) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

size_t fmha_decode_static_scratch_bytes() { return kStaticScratchBytes; }

static hipError_t static_scratch_ptr(char** out) {
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
    *out = static_cast<char*>(p);
    return hipSuccess;
}

template <typename T, int WAVES, int NSTAGE>
static hipError_t launch_decode(const T* Q, const T* K, const T* V, T* O, float* LSE, float* part, unsigned* counters, int B,
                                int Hq, int Hkv, int Sq, int Sk, float scale_log2, int causal, int kv_valid, int splits,
                                int tiles_per_split, long workgroups, const FmhaStrides& sd, hipStream_t stream) {
    constexpr int LDS = WAVES * NSTAGE * dec::STAGE_BYTES;
    static_assert(LDS >= WAVES * (32 * dec::D + 64) * 4 + 64, "the combine step reuses the pipeline memory");
    static_assert(LDS >= (3 * dec::kMaxSplits * 32 + 32 + 64) * 4, "so does the merge of the key ranges");
    auto kern = fmha_decode_kernel<T, WAVES, NSTAGE>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), LDS); e != hipSuccess) return e;
    if (workgroups > 0x7fffffffL) return hipErrorInvalidValue;
    kern<<<dim3((unsigned)workgroups), dim3(WAVES * 64), LDS, stream>>>(Q, K, V, O, LSE, part, counters, B, Hq, Hkv, Sq, Sk, scale_log2,
                                                                         causal, kv_valid, splits, tiles_per_split, sd);
    return hipGetLastError();
}

template <typename T>
hipError_t fmha_decode_dispatch(const T* Q, const T* K, const T* V, T* O, float* LSE, int B, int Hq,
                                int Hkv, int Sq, int Sk, float scale, int causal, int kv_valid, const FmhaStrides& sd,
                                const FmhaWorkspace& ws, hipStream_t stream) {
    using namespace dec;
    const DecodePlan plan = decode_plan(B, Hq, Hkv, Sq, kv_valid);
    char* wsp = nullptr;
    hipError_t e = hipSuccess;
    if (plan.bytes > 0) {
        // Ticket counters must be zero when the kernel starts. The library's buffers and the static array are zeroed once
        // (a fresh buffer by the fill kernel below, the static array by the loader) and every call leaves its counters at
        // zero; a caller's memory holds anything, so its counters are zeroed on every call.
        bool clear_counters = false;
        long n_counters = (long)B * Hkv * kCounterStride;   // this call's counters
        switch (ws.kind) {
            case FmhaWorkspace::kCaller:
                if (ws.ptr == nullptr || ws.bytes < plan.bytes || reinterpret_cast<uintptr_t>(ws.ptr) % 16 != 0) return hipErrorInvalidValue;
                wsp = static_cast<char*>(ws.ptr);
                clear_counters = true;
                break;
            case FmhaWorkspace::kStatic:
                if (plan.bytes > kStaticScratchBytes) return hipErrorOutOfMemory;   // the entry point checks first and says why
                e = static_scratch_ptr(&wsp);
                break;
            default:
                e = decode_workspace(plan.bytes, stream, &wsp, &clear_counters);
                n_counters = kCounterBytes / (long)sizeof(unsigned);   // a fresh buffer: the whole counter region, once
                break;
        }
        if (e != hipSuccess) return e;
        if (clear_counters) {
            fmha_decode_clear_kernel<<<dim3(4), dim3(256), 0, stream>>>(reinterpret_cast<unsigned*>(wsp), (int)n_counters);
            e = hipGetLastError();
        }
        if (e != hipSuccess) return e;
    }
    float* part = reinterpret_cast<float*>(wsp + plan.counter_bytes);
    unsigned* counters = reinterpret_cast<unsigned*>(wsp);
    const float scale_log2 = scale * 1.4426950408889634f;
    return launch_decode<T, 4, 2>(Q, K, V, O, LSE, part, counters, B, Hq, Hkv, Sq, Sk, scale_log2, causal, kv_valid, plan.splits,
                                  plan.tiles_per_split, plan.workgroups, sd, stream);
}

template hipError_t fmha_decode_dispatch<half_t>(const half_t*, const half_t*, const half_t*, half_t*, float*, int, int, int, int,
                                                  int, float, int, int, const FmhaStrides&, const FmhaWorkspace&, hipStream_t);
template hipError_t fmha_decode_dispatch<bf16_t>(const bf16_t*, const bf16_t*, const bf16_t*, bf16_t*, float*, int, int, int, int,
                                                 int, float, int, int, const FmhaStrides&, const FmhaWorkspace&, hipStream_t);

}  // namespace mi355

#ifdef MI355_TIMELINE
// profiling build: copies the records of the last generation-step attention launch to the host
extern "C" int mi355_timeline_read_fmha_decode(void* dst, size_t bytes) {
    const size_t all = sizeof(unsigned long long) * mi355::timeline::kMaxWorkgroups * mi355::timeline::kSlots;
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(mi355::fmha_decode_stamps), bytes < all ? bytes : all);
}
#endif
