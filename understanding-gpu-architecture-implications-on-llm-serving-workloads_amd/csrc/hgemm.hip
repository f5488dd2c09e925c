// fp16 GEMM for gfx950 (MI355X): C[M,N] = op(A) * op(B), fp16 operands, fp32 accumulation in the MFMA
// accumulators, one rounding to fp16 on the store.
//
// Replaces the reference's GEMM ladder (kernels/gemm/pkg/gemm_unified/csrc/{auto,semi,manual}/gemm_*.{cu,cpp});
// the three operand layouts are the ones the reference's op indices use
// (kernels/gemm/test/correct.py:9-15): NN for finegemm_0..11, TN (a stored [K,M]) for 12/16 and NT (b stored
// [N,K]) for 13..15.
//
// Main kernel: one workgroup of 8 waves computes a 256x256 tile of C, K is walked in steps of 64.
//   * global -> LDS staging uses 16-byte direct-to-LDS copies (no VGPR bounce) into a ring of stages (two 64 KiB
//     stages for the 256x256 tile, three for 128x128, five for 64x128 / 128x64, eight - or four, with two workgroups
//     on a CU - for 64x64); every wave-instruction writes 1 KiB of contiguous LDS, the XOR swizzle is applied on the
//     global-address side.
//     The copies are buffer loads (scalar tile base + one 32-bit lane offset): a global load with 64-bit lane
//     addresses takes about twice as much issue time away from the MFMAs it runs beside, and several times as
//     much when such loads are issued back to back.
//   * a wave issues an instruction every ~5 cycles at best and every ~10 next to its SIMD partner's MFMAs, whatever the
//     instruction, so the K loop is kept short: it is unrolled over the ring, which makes every LDS address a
//     loop-invariant register plus an immediate (A's stages lie one behind the other, then B's, so that one register
//     reaches all stages of an operand) and every copy destination a scalar plus an immediate; the tile bases advance
//     inside their buffer resources; every tile issues the same instructions (the copies of the last tiles run on a
//     resource whose size is set to zero: out of range, nothing is fetched), so the waits never change and the loop has
//     one body per stage. Per K tile and wave of the 256x256 kernel: 64 MFMAs and ~58 other instructions.
//   * K is any multiple of 8: the tile that holds the last K % 64 columns is taken first, by the prologue, whose copies
//     point the lanes at k >= K out of the resource's range (such a copy writes zeros to LDS); the loop is the same code
//     for every K.
//   * an operand whose K index is contiguous in memory is read from LDS with ds_read_b128; an operand whose
//     M/N index is contiguous (B in the NN case) is read with the transposing ds_read_b64_tr_b16, so no
//     transpose pass over B is ever made.
//   * each wave owns a 128x64 sub-tile = 8x4 MFMA 16x16x32 blocks (128 fp32 accumulators per lane); with random
//     operands the 16x16x32 instruction sustains a ~14 % higher rate than 32x32x16 under the board's power limit.
//     The MFMA is issued with the B fragment as first operand, i.e. it produces the transposed block, so a
//     lane ends up with 4 consecutive N of one row of C; the epilogue parks the sub-tile in LDS and stores whole
//     128-byte lines.
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>
#include "mi355_common.h"
#include "mi355_serving_internal.h"
#include "mi355_timeline.h"

namespace mi355 {

// profiling build: per workgroup of hgemm_main_kernel [wall: entry, loop start, loop end, exit; cycles: loop start, loop
// end; K tiles; 0]
MI355_TL(static __device__ unsigned long long hgemm_stamps[timeline::kMaxWorkgroups * timeline::kSlots];)

// ---------------------------------------------------------------------------------------------------------
// LDS tile descriptions
// ---------------------------------------------------------------------------------------------------------

// Operand tile whose K index is contiguous in memory: LDS holds [ROWS][BK] halfs, row = M (or N) index.
// 16-byte chunk c of row r lives at chunk position c ^ swz(r).
template <int ROWS, int BK, int NWAVES>
struct KContigTile {
    static constexpr int kChunksPerRow = BK / 8;
    static constexpr int kRowBytes = BK * 2;
    static constexpr int kRowsPerInst = 64 / kChunksPerRow;
    static constexpr int kRowsPerPass = kRowsPerInst * NWAVES;
    static constexpr int kInsts = ROWS / kRowsPerPass;
    static constexpr int kBytes = ROWS * kRowBytes;
    static_assert(ROWS % kRowsPerPass == 0, "tile rows must be a multiple of one pass of the workgroup");
    static_assert(BK == 64, "swizzle below is written for 128-byte rows");

    // A fragment read (ds_read_b128) has lane l at row l % 16, chunk c0 + l / 16. Rows of equal parity share the same
    // half of the 256-byte bank window, so their chunk positions must differ: over 16 consecutive lanes (16 rows, one
    // chunk), and over the lanes l and l + 32 that the hardware serves together (8 rows, chunks c and c + 2, i.e. c ^ 2).
    // Bits 0 and 2 of the XOR value tell the 4 rows of one parity inside an 8-row group apart, bit 1 the two groups.
    __device__ static __forceinline__ int swz(int row) {
        return ((row >> 1) & 1) | (((row >> 2) & 1) << 2) | (((row >> 3) & 1) << 1);
    }

    // element offset (in halfs, relative to the tile origin in global memory) of this lane's first copy
    __device__ static __forceinline__ long first_copy_offset(int wave, int lane, long ld) {
        int row = wave * kRowsPerInst + lane / kChunksPerRow;
        int chunk = (lane % kChunksPerRow) ^ swz(row);
        return (long)row * ld + chunk * 8;
    }
    __device__ static __forceinline__ long copy_stride(long ld) { return (long)kRowsPerPass * ld; }
    __device__ static __forceinline__ long ktile_stride(long /*ld*/) { return BK; }
    __device__ static __forceinline__ int lds_inst_offset(int inst, int wave) { return (inst * NWAVES + wave) * 1024; }

    // byte offset inside the tile of this lane's 16 bytes of the fragment (16 rows x 32 k) for k-substep kk, first
    // row row0 (a multiple of 16): lane l holds k = 32 kk + 8 (l / 16) .. +7 of row l % 16
    __device__ static __forceinline__ int frag_offset(int row0, int kk, int lane) {
        int row = row0 + (lane & 15);
        int chunk = (kk * 4 + (lane >> 4)) ^ swz(row);
        return row * kRowBytes + chunk * 16;
    }
};

// Operand tile whose M/N index is contiguous in memory: LDS holds [BK][COLS] halfs, row = K index.
template <int COLS, int BK, int NWAVES>
struct MNContigTile {
    static constexpr int kChunksPerRow = COLS / 8;
    static constexpr int kRowBytes = COLS * 2;
    static constexpr int kRowsPerInst = 64 / kChunksPerRow;
    static constexpr int kRowsPerPass = kRowsPerInst * NWAVES;
    static constexpr int kInsts = BK / kRowsPerPass;
    static constexpr int kBytes = BK * kRowBytes;
    static_assert(COLS == 256 || COLS == 128 || COLS == 64, "the swizzles below are written for these row lengths");
    static_assert(kRowsPerPass % 16 == 0, "copy i of a lane is 16 rows or a multiple further down: same swizzle for all i");
    static_assert(BK % kRowsPerPass == 0, "tile depth must be a multiple of one pass of the workgroup");

    // A transposing read touches, per 16 lanes, 4 k-rows x 32 bytes (two neighbouring chunks); lanes 0..31 of a
    // fragment read cover rows {0..3} and {8..11} (+ a multiple of 4 that does not change what follows). XOR-ing the
    // chunk index with an even number that differs for those 8 rows keeps their 8 chunk pairs on distinct banks.
    // Rows of 128 bytes (COLS == 64) fill only half of the 256-byte bank window: rows of equal parity share a half, so
    // it is the 4 rows of one parity among those 8 that need distinct chunk pairs (bits 1 and 3 of the row tell them apart).
    __device__ static __forceinline__ int swz(int row) {
        if constexpr (COLS == 64) return (((row >> 1) & 1) | (((row >> 3) & 1) << 1)) << 1;
        else return ((row & 3) | (((row >> 3) & 1) << 2)) << 1;
    }
    __device__ static __forceinline__ long first_copy_offset(int wave, int lane, long ld) {
        int row = wave * kRowsPerInst + lane / kChunksPerRow;
        int chunk = (lane % kChunksPerRow) ^ swz(row);
        return (long)row * ld + chunk * 8;
    }
    __device__ static __forceinline__ long copy_stride(long ld) { return (long)kRowsPerPass * ld; }
    __device__ static __forceinline__ long ktile_stride(long ld) { return (long)BK * ld; }
    __device__ static __forceinline__ int lds_inst_offset(int inst, int wave) { return (inst * NWAVES + wave) * 1024; }

    // byte offset of this lane's transposing read for the fragment (32 k x 16 cols) whose first column is col0 (a
    // multiple of 16): group g = lane / 16 reads k rows 8g .. 8g+3, input lane j of the group supplies the 4 columns
    // 4 (j % 4) .. +3 of row j / 4. Add (kk*32 + 4*t) * kRowBytes for substep kk and half t (neither changes swz).
    __device__ static __forceinline__ int frag_offset(int col0, int lane) {
        int j = lane & 15;
        int row = 8 * (lane >> 4) + (j >> 2);
        int chunk = (col0 >> 3) + ((j & 3) >> 1);
        return row * kRowBytes + ((chunk ^ swz(row)) << 4) + (j & 1) * 8;
    }
};

// ---------------------------------------------------------------------------------------------------------
// 256x256x64 main kernel
// ---------------------------------------------------------------------------------------------------------

template <bool A_KC, bool B_KC, int BM_, int BN_, int WM_, int WN_, int STAGES = 0>
struct MainCfg {
    static constexpr int BM = BM_, BN = BN_, BK = 64;
    static constexpr int WM = WM_, WN = WN_, NWAVES = WM_ * WN_, NTHREADS = NWAVES * 64;
    static constexpr int TM = BM / WM / 16;  // MFMA 16x16 blocks along M per wave
    static constexpr int TN = BN / WN / 16;  // along N
    // (the description of the layout an operand does not have is never used: it is formed with an extent that exists)
    using ATileK = KContigTile<A_KC ? BM : 256, BK, NWAVES>;
    using ATileM = MNContigTile<A_KC ? 64 : BM, BK, NWAVES>;
    using BTileK = KContigTile<B_KC ? BN : 256, BK, NWAVES>;
    using BTileN = MNContigTile<B_KC ? 64 : BN, BK, NWAVES>;
    static constexpr int A_BYTES = BM * BK * 2;
    static constexpr int B_BYTES = BN * BK * 2;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    // 64 KiB stages: two of them fit; the 48 KiB stages of the 128x256 tiles and the 32 KiB stages of the 128x128 tile
    // get a third, which gives every copy one more K tile of time to land (small problems run few tiles per workgroup and are bound by that latency). The narrow tiles
    // serve products with few rows, which are bound by the stream of the weight matrix from HBM: their ring is as deep
    // as 128 KiB of LDS allow (5 stages of 24 KiB, 8 of 16 KiB), so that a CU keeps ~50 KiB of that stream in flight.
    // STAGES > 0 sets the depth (the 64x64 tiles of small products run with four stages, two workgroups to a CU).
    static constexpr int NSTAGE = STAGES > 0 ? STAGES : STAGE_BYTES > 48 * 1024 ? 2 : STAGE_BYTES > 24 * 1024 ? 3 : STAGE_BYTES > 16 * 1024 ? 5 : 8;
    static constexpr int LDS_BYTES = STAGE_BYTES * NSTAGE;
    static constexpr int A_INSTS = A_BYTES / (NWAVES * 1024);  // 16-byte copies per lane per K tile
    static constexpr int B_INSTS = B_BYTES / (NWAVES * 1024);
    static constexpr int FRAG_SLOTS = TM > TN ? TM : TN;
};

// x < 0 ? -1 : 0 of a wave-uniform value, computed and kept on the scalar unit (written as a shift or a select, the
// compiler may carry the result, and every value formed from it, in vector registers)
__device__ __forceinline__ int sign_mask_scalar(int x) {
    int r;
    asm("s_ashr_i32 %0, %1, 31" : "=s"(r) : "s"(x) : "scc");
    return r;
}

// f(std::integral_constant<int, I>) for I = BEGIN .. END-1, unrolled at compile time
template <int BEGIN, int END, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + 1, END>(f);
    }
}

// Map the linear workgroup id to a C tile so that the workgroups resident on one XCD (ids congruent mod 8)
// cover a compact rectangle of tiles: they then share A row-panels and B column-panels in that XCD's L2.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    constexpr int kXcd = 8;
    // Large grids: the 256 workgroups that run at the same time (ids 256 s .. 256 s + 255, one per CU) take one
    // super-block of 256 tiles, each XCD an 8 x 4 piece of it, and the super-blocks follow one another in serpentine
    // order, so that consecutive ones share their row panels of A or their column panels of B. A super-block reads
    // (16 + 16) or (32 + 8) panels where the same 256 tiles taken as 8 stripes of 8 x 4 from all over the matrix read
    // all 32 row panels: fewer bytes pass through the memory-side cache, and half of them were there a step earlier.
    const int sb_n = tiles_n % 16 == 0 ? 16 : tiles_n % 8 == 0 ? 8 : 0;   // super-block: sb_m x sb_n tiles
    const int sb_m = sb_n ? 256 / sb_n : 0;
    if (sb_n && tiles_m % sb_m == 0 && total >= 512) {
        const int step = bid >> 8, x = bid & 7, j = (bid >> 3) & 31;    // j: this XCD's 32 workgroups of the step
        const int blocks_n = tiles_n / sb_n;
        const int brow = step / blocks_n;
        const int bcol = (brow & 1) ? blocks_n - 1 - step % blocks_n : step % blocks_n;
        const int xcd_cols = sb_n / 4;                                   // XCD pieces side by side in a super-block
        tm = brow * sb_m + (x / xcd_cols) * 8 + (j & 7);
        tn = bcol * sb_n + (x % xcd_cols) * 4 + (j >> 3);
        return;
    }
    int t = bid;
    if (total % kXcd == 0) {
        int per = total / kXcd;
        t = (bid % kXcd) * per + bid / kXcd;
    }
    // grouped ordering: walk down GROUP rows of tiles before moving to the next column
    constexpr int GROUP = 8;
    int group_size = GROUP * tiles_n;
    int g = t / group_size;
    int first_m = g * GROUP;
    int rows = min(GROUP, tiles_m - first_m);
    int in_g = t - g * group_size;
    tm = first_m + in_g % rows;
    tn = in_g / rows;
}

// Epilogue of the tiled kernels for one wave's sub-tile of TM x TN blocks of 16x16 (first row row0, first stored column
// col0, of a C with NC columns). A lane holds C[m][n .. n+3] for m = l%16, n = 4*(l/16) of every block. Storing that
// directly would write 8-byte pieces of 16 different rows per instruction (partial cache lines, read-modify-write in
// the memory system), so the wave first parks its sub-tile in its own slice of LDS (cst; fp16, 16-byte chunks
// XOR-swizzled by row) and then stores whole rows: every store instruction writes complete 128-byte lines.
// EPI == 1: the wave's columns come in groups of [32 gate | 32 up]; output block jo takes its gate from block
// 4 (jo / 2) + jo % 2 and its up from two blocks further.
template <typename T, int TM, int TN, int EPI, bool RAGGED>
__device__ __forceinline__ void store_wave_tile(const float4v (&acc)[TM][TN], MI355_LDS char* cst, T* C, const T* R, long row0,
                                                long col0, int M, int NC, long ldc, long ldr, int lane) {
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    static_assert(EPI == 0 || TN % 4 == 0, "the gate/up epilogue pairs column blocks 32 columns apart");
    constexpr int TNO = EPI == 1 ? TN / 2 : TN;   // column blocks a wave stores
    constexpr int kRowHalfs = TNO * 16;           // width of the stored wave sub-tile
    constexpr int kRowBytesC = kRowHalfs * 2;
    constexpr int kChunksC = kRowBytesC / 16;     // 16-byte chunks per row (4, 8 or 16)
    constexpr int kRowsPerStore = 64 / kChunksC;  // rows covered by one store instruction
    constexpr int kSwzC = kChunksC < 8 ? kChunksC - 1 : 7;
    {
        const int r = lane & 15;
        const int g = lane >> 4;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row = i * 16 + r;
#pragma unroll
            for (int jo = 0; jo < TNO; ++jo) {
                V4 v;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if constexpr (EPI == 1) {
                        const int gj = (jo / 2) * 4 + (jo % 2);
                        const float gt = acc[i][gj][q];
                        const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-gt * 1.4426950408889634f));
                        v[q] = (T)(gt * sig * acc[i][gj + 2][q]);
                    } else {
                        v[q] = (T)acc[i][jo][q];
                    }
                }
                const int chunk = (2 * jo + (g >> 1)) ^ (row & kSwzC);
                *(MI355_LDS V4*)(cst + row * kRowBytesC + chunk * 16 + (g & 1) * 8) = v;
            }
        }
    }
    // only this wave reads what it wrote: no workgroup barrier needed, the LDS operations of a wave complete in order
    {
        const int rr = lane / kChunksC;
        const int cc = lane % kChunksC;
        T* cbase = C + row0 * ldc + col0 + cc * 8;
        const long rows_left = M - row0;   // RAGGED: rows and columns that exist
        const long cols_left = NC - (col0 + cc * 8);   // of this lane's 8
        const T* rbase = R + row0 * ldr + col0 + cc * 8;
#pragma unroll
        for (int it = 0; it < TM * 16 / kRowsPerStore; ++it) {
            const int row = it * kRowsPerStore + rr;
            V8 v = *(MI355_LDS const V8*)(cst + row * kRowBytesC + ((cc ^ (row & kSwzC)) << 4));
            if constexpr (!RAGGED) {
                if (R != nullptr) {
                    const V8 r = *(const V8*)(rbase + (long)row * ldr);
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = (T)((float)v[j] + (float)r[j]);
                }
                *(V8*)(cbase + (long)row * ldc) = v;
            } else if (row < rows_left && cols_left >= 8) {
                // C's rows (and the residual's) may start at any element: the 16 bytes move as a copy of no stated
                // alignment, for which the compiler still issues one 16-byte access (global memory takes unaligned ones)
                if (R != nullptr) {
                    V8 r;
                    __builtin_memcpy(&r, rbase + (long)row * ldr, 16);
#pragma unroll
                    for (int j = 0; j < 8; ++j) v[j] = (T)((float)v[j] + (float)r[j]);
                }
                __builtin_memcpy(cbase + (long)row * ldc, &v, 16);
            } else if (row < rows_left) {
                // the last columns of a C whose width is not a multiple of 8: element by element
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (j < cols_left) {
                        T x = v[j];
                        if (R != nullptr) x = (T)((float)x + (float)rbase[(long)row * ldr + j]);
                        cbase[(long)row * ldc + j] = x;
                    }
            }
        }
    }
}

// EPI selects what is stored: 0 = the product; 1 = silu(g) * u for a B operand whose columns alternate between 32 gate
// columns and their 32 up columns (`act_fn(gate_proj(x)) * up_proj(x)`, benchmarks/flashattn-cuda/modeling_llama.py:227,
// with the two projections interleaved in one weight matrix): a wave then holds g and u of the same outputs in its two
// column blocks, at the same accumulator positions, and C has N / 2 columns.
// R (may be null, may be C itself): a residual of C's shape added to the rounded product, `residual + proj(x)` of
// modeling_llama.py:776,781 with the rounding of the unfused sequence (product to T, then the sum to T).
// RAGGED: M and N need not be multiples of the tile, nor of 8. Copies of rows past the end are redirected to the last row
// (or, for an operand whose M/N index is contiguous, to the last 8 columns of its extent rounded up to a multiple of 8: the
// columns between the extent and that multiple lie in the padding of the operand's rows, because its leading dimension is
// a multiple of 8, and what they hold only reaches rows / columns of the product that are never stored), so every load
// stays inside the matrices' rows; the epilogue stores only what exists: whole 16-byte pieces wherever a row of C starts
// (global memory takes such an access at any element), the last N % 8 columns of a row element by element.
// SPLIT_K: the grid's y index selects one of `splits` equal ranges of K (K a multiple of 64 * splits). A workgroup
// stores its partial tile (fp32, each lane its own accumulators) to `part`, draws a ticket from the tile's counter, and
// the workgroup that draws the last one adds the partial tiles of all ranges, in the order of the ranges (so the sum does
// not depend on which workgroup arrives last), and runs the epilogue. Ordering without a fence, as in the split-KV
// attention kernel: the partial tiles are stored device-coherently (`sc1`), every lane waits for its stores to be
// acknowledged (`s_waitcnt vmcnt(0)`), a workgroup barrier, then one thread draws the ticket with a relaxed device-scope
// atomic (carried out at the memory side); the last workgroup reads the partial tiles with `sc1` loads behind the branch
// on the ticket's value, and sets the counter back to zero for the next launch.
template <typename T, bool A_KC, bool B_KC, int BM, int BN, int WM, int WN, int EPI = 0, bool RAGGED = false, int STAGES = 0, int PER_CU = 1,
          bool SPLIT_K = false>
__global__ __launch_bounds__(WM * WN * 64) __attribute__((amdgpu_waves_per_eu(WM * WN / 4, PER_CU * WM * WN / 4)))
void hgemm_main_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                         T* C, const T* R, int M, int N, int K, long lda,
                                                         long ldb, long ldc, long ldr, float* part, unsigned* counters, int splits) {
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    using V2 = typename Elem<T>::v2;
    using Cfg = MainCfg<A_KC, B_KC, BM, BN, WM, WN, STAGES>;
    using ATK = typename Cfg::ATileK;
    using ATM = typename Cfg::ATileM;
    using BTK = typename Cfg::BTileK;
    using BTN = typename Cfg::BTileN;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, BK = Cfg::BK;

    MI355_TL(unsigned long long tl_w[4] = {timeline::wall_clock(), 0, 0, 0}; unsigned long long tl_c[2] = {0, 0};)
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / Cfg::WN;
    const int wn = wave % Cfg::WN;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, (M + Cfg::BM - 1) / Cfg::BM, (N + Cfg::BN - 1) / Cfg::BN, tile_m, tile_n);
    const long m0 = (long)tile_m * Cfg::BM;
    const long n0 = (long)tile_n * Cfg::BN;
    if constexpr (SPLIT_K) {   // this workgroup's range of K
        K /= splits;
        const long k0 = (long)blockIdx.y * K;
        A += A_KC ? k0 : k0 * lda;
        B += B_KC ? k0 : k0 * ldb;
    }

    // ---- global -> LDS copy descriptors --------------------------------------------------------------
    // A copy reads (tile base, kept in scalar registers and advanced per K tile) + (this lane's byte offset inside the
    // tile, a loop-invariant 32-bit VGPR) + (copy index * uniform step). Offsets inside a tile fit 32 bits because the
    // launcher only takes leading dimensions below 2^22 elements.
    const char* a_base;
    const char* b_base;
    uint32_t a_lane_off, b_lane_off, a_copy_step, b_copy_step;
    long a_k_step, b_k_step;
    if constexpr (A_KC) {  // A stored [M,K]
        a_base = (const char*)(A + m0 * lda);
        a_lane_off = (uint32_t)(ATK::first_copy_offset(wave, lane, lda) * 2);
        a_copy_step = (uint32_t)(ATK::copy_stride(lda) * 2);
        a_k_step = ATK::ktile_stride(lda) * 2;
    } else {  // A stored [K,M]
        a_base = (const char*)(A + m0);
        a_lane_off = (uint32_t)(ATM::first_copy_offset(wave, lane, lda) * 2);
        a_copy_step = (uint32_t)(ATM::copy_stride(lda) * 2);
        a_k_step = ATM::ktile_stride(lda) * 2;
    }
    if constexpr (B_KC) {  // B stored [N,K]
        b_base = (const char*)(B + n0 * ldb);
        b_lane_off = (uint32_t)(BTK::first_copy_offset(wave, lane, ldb) * 2);
        b_copy_step = (uint32_t)(BTK::copy_stride(ldb) * 2);
        b_k_step = BTK::ktile_stride(ldb) * 2;
    } else {  // B stored [K,N]
        b_base = (const char*)(B + n0);
        b_lane_off = (uint32_t)(BTN::first_copy_offset(wave, lane, ldb) * 2);
        b_copy_step = (uint32_t)(BTN::copy_stride(ldb) * 2);
        b_k_step = BTN::ktile_stride(ldb) * 2;
    }

    // RAGGED: one lane offset per copy, rows / column chunks past the end folded back inside the matrix (never in
    // front of the tile origin: the tile exists, so its first row and its first 8 columns do)
    uint32_t a_voff[RAGGED ? Cfg::A_INSTS : 1];
    uint32_t b_voff[RAGGED ? Cfg::B_INSTS : 1];
    if constexpr (RAGGED) {
        // byte offset from the tile base of copy i of this lane; origin / extent along the tile's M (or N) axis
        auto clamped = [&](long ld, bool k_contig, int rows_per_inst, int chunks_per_row, int rows_per_pass, int i,
                           long origin, long extent, int swz) {
            const int row = wave * rows_per_inst + lane / chunks_per_row + i * rows_per_pass;
            const int chunk = (lane % chunks_per_row) ^ swz;
            if (k_contig) return (uint32_t)(((min(origin + row, extent - 1) - origin) * ld + chunk * 8) * 2);   // row = M/N index
            return (uint32_t)(((long)row * ld + min(origin + chunk * 8, extent - 8) - origin) * 2);              // row = K index
        };
#pragma unroll
        for (int i = 0; i < Cfg::A_INSTS; ++i) {
            if constexpr (A_KC) {
                const int row = wave * ATK::kRowsPerInst + lane / ATK::kChunksPerRow;
                a_voff[i] = clamped(lda, true, ATK::kRowsPerInst, ATK::kChunksPerRow, ATK::kRowsPerPass, i, m0, M, ATK::swz(row));
            } else {
                const int row = wave * ATM::kRowsPerInst + lane / ATM::kChunksPerRow + i * ATM::kRowsPerPass;
                a_voff[i] = clamped(lda, false, ATM::kRowsPerInst, ATM::kChunksPerRow, ATM::kRowsPerPass, i, m0, (M + 7) & ~7, ATM::swz(row));
            }
        }
#pragma unroll
        for (int i = 0; i < Cfg::B_INSTS; ++i) {
            if constexpr (B_KC) {
                const int row = wave * BTK::kRowsPerInst + lane / BTK::kChunksPerRow;
                b_voff[i] = clamped(ldb, true, BTK::kRowsPerInst, BTK::kChunksPerRow, BTK::kRowsPerPass, i, n0, N, BTK::swz(row));
            } else {
                const int row = wave * BTN::kRowsPerInst + lane / BTN::kChunksPerRow + i * BTN::kRowsPerPass;
                b_voff[i] = clamped(ldb, false, BTN::kRowsPerInst, BTN::kChunksPerRow, BTN::kRowsPerPass, i, n0, (N + 7) & ~7, BTN::swz(row));
            }
        }
    }
    // K need not be a multiple of the tile depth: the last K tile, which then holds K % 64 columns (rows) of the
    // operands, is taken FIRST, by the prologue, with copies of its own (below); the loop never sees it.
    const int ktiles = (K + BK - 1) / BK;
    const int k_first = K - (ktiles - 1) * BK;   // depth of that tile: 8 .. 64
    const long first_tile = k_first < BK ? ktiles - 1 : 0;   // position along K, in tiles, of the tile taken first
    int4v a_res = make_buffer_resource(a_base + first_tile * a_k_step);
    int4v b_res = make_buffer_resource(b_base + first_tile * b_k_step);

    // ---- LDS fragment read offsets (bytes inside one stage) -------------------------------------------
    // A fragments: TM blocks of 16 rows; B fragments: TN blocks of 16 columns; a K tile is two 32-deep substeps.
    constexpr int NSUB = BK / 32;
    static_assert(NSUB == 2, "the pipeline below is written for two substeps per K tile");
    // LDS layout: the NSTAGE stages of A one behind the other, then those of B. A stage index is a compile-time constant
    // wherever fragments are read (the K loop is unrolled over the ring), so a fragment address is a loop-invariant
    // register plus an immediate offset and the loop holds no address arithmetic. The immediate field of an LDS read
    // reaches 64 KiB: where an operand's ring is longer than that (less the largest offset inside a stage), its stages
    // are grouped into sets within reach, one register per set.
    constexpr int kAImm = A_KC ? (TM - 1) * 16 * ATK::kRowBytes : 36 * ATM::kRowBytes;   // largest offset inside a stage
    constexpr int kBImm = B_KC ? (TN - 1) * 16 * BTK::kRowBytes : 36 * BTN::kRowBytes;
    constexpr int kAPerSet = (65535 - kAImm) / Cfg::A_BYTES + 1, kBPerSet = (65535 - kBImm) / Cfg::B_BYTES + 1;
    constexpr int kASets = (Cfg::NSTAGE + kAPerSet - 1) / kAPerSet, kBSets = (Cfg::NSTAGE + kBPerSet - 1) / kBPerSet;
    constexpr int kBRegion = Cfg::NSTAGE * Cfg::A_BYTES;
    MI355_LDS char* a_ptr[kASets][Cfg::FRAG_SLOTS];  // K-contiguous operand: one per k-substep; M/N-contiguous: one per 16-wide block
    MI355_LDS char* b_ptr[kBSets][Cfg::FRAG_SLOTS];
#pragma unroll
    for (int s = 0; s < kASets; ++s) {
        MI355_LDS char* base = smem + s * kAPerSet * Cfg::A_BYTES;
        if constexpr (A_KC) {
#pragma unroll
            for (int kk = 0; kk < NSUB; ++kk) a_ptr[s][kk] = base + ATK::frag_offset(wm * TM * 16, kk, lane);
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i) a_ptr[s][i] = base + ATM::frag_offset(wm * TM * 16 + i * 16, lane);
        }
    }
#pragma unroll
    for (int s = 0; s < kBSets; ++s) {
        MI355_LDS char* base = smem + kBRegion + s * kBPerSet * Cfg::B_BYTES;
        if constexpr (B_KC) {
#pragma unroll
            for (int kk = 0; kk < NSUB; ++kk) b_ptr[s][kk] = base + BTK::frag_offset(wn * TN * 16, kk, lane);
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j) b_ptr[s][j] = base + BTN::frag_offset(wn * TN * 16 + j * 16, lane);
        }
    }

    float4v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

    // Software pipeline, pinned slot by slot (a slot = one MFMA 16x16x32 and what is issued in its shadow;
    // sched_barrier keeps the compiler from moving anything between slots):
    //   * the fragments of the next substep are read during the FIRST slots of the current one, in the order the MFMAs
    //     will need them, so they have landed long before that substep ends and no MFMA waits on a read it has just
    //     issued;
    //   * the barrier that hands over the next K tile sits in front of the last substep: the reads of that substep
    //     were issued a substep earlier, so the wave reaches the barrier with nothing in flight, and goes on with
    //     MFMAs whose operands are already in registers;
    //   * the copies of the tile after next go out during that last substep, spread over its slots, behind the reads of
    //     the next tile's first fragments.
    constexpr int NSLOT = TM * TN;
    constexpr int NFRAG = TM + TN;
    constexpr int NCOPY = Cfg::A_INSTS + Cfg::B_INSTS;
    // fragment f of substep kk, f in the order of first use: A0, B0 .. B(TN-1), A1 .. A(TM-1)
    auto load_frag = [&](auto sc, auto kc, auto fc, V8(&afn)[TM], V8(&bfn)[TN]) {
        constexpr int f = decltype(fc)::value, kk = decltype(kc)::value;
        constexpr int st = decltype(sc)::value;
        constexpr int aset = st / kAPerSet, ao = (st % kAPerSet) * Cfg::A_BYTES;   // set, and stage offset inside it
        constexpr int bset = st / kBPerSet, bo = (st % kBPerSet) * Cfg::B_BYTES;
        if constexpr (f == 0 || f > TN) {
            constexpr int i = f == 0 ? 0 : f - TN;
            if constexpr (A_KC) {
                afn[i] = Elem<T>::frag(lds_read_b128(a_ptr[aset][kk] + (ao + i * 16 * ATK::kRowBytes)));
            } else {
                half4 lo = lds_read_tr16_b64(a_ptr[aset][i] + (ao + (kk * 32) * ATM::kRowBytes));
                half4 hi = lds_read_tr16_b64(a_ptr[aset][i] + (ao + (kk * 32 + 4) * ATM::kRowBytes));
                afn[i] = Elem<T>::frag(concat(lo, hi));
            }
        } else {
            constexpr int j = f - 1;
            if constexpr (B_KC) {
                bfn[j] = Elem<T>::frag(lds_read_b128(b_ptr[bset][kk] + (bo + j * 16 * BTK::kRowBytes)));
            } else {
                half4 lo = lds_read_tr16_b64(b_ptr[bset][j] + (bo + (kk * 32) * BTN::kRowBytes));
                half4 hi = lds_read_tr16_b64(b_ptr[bset][j] + (bo + (kk * 32 + 4) * BTN::kRowBytes));
                bfn[j] = Elem<T>::frag(concat(lo, hi));
            }
        }
    };
    auto load_frags = [&](auto sc, auto kc, V8(&afn)[TM], V8(&bfn)[TN]) {
        static_for<0, NFRAG>([&](auto fc) { load_frag(sc, kc, fc, afn, bfn); });
    };
    // copy d of a stage lands at (stage, operand, d) + this wave's 1 KiB slice: a scalar register plus an immediate
    const uint32_t wave_lds = (uint32_t)(uintptr_t)(smem + wave * 1024);
    // part selects what is issued: 0 = the whole copy, 1 = only the scalar instruction that points M0 at the destination,
    // 2 = only the load (M0 was set a slot earlier, the matrix instruction in between is the wait state M0 needs)
    auto issue_copy = [&](auto sc, auto dc, auto part) {
        constexpr int d = decltype(dc)::value, pt = decltype(part)::value;
        constexpr int st = decltype(sc)::value;
        constexpr bool is_a = d < Cfg::A_INSTS;
        constexpr int e = is_a ? d : d - Cfg::A_INSTS;
        constexpr int dst = is_a ? st * Cfg::A_BYTES + e * Cfg::NWAVES * 1024 : kBRegion + st * Cfg::B_BYTES + e * Cfg::NWAVES * 1024;
        if constexpr (pt == 1) {
            set_m0_at<dst>(wave_lds);
        } else {
            const int4v& res = is_a ? a_res : b_res;
            uint32_t voff, soff = 0u;
            if constexpr (RAGGED && is_a) voff = a_voff[e];
            else if constexpr (RAGGED) voff = b_voff[e];
            else { voff = is_a ? a_lane_off : b_lane_off; soff = e * (is_a ? a_copy_step : b_copy_step); }
            if constexpr (pt == 0) copy16_buffer_to_lds_at<dst>(res, voff, soff, wave_lds);
            else copy16_buffer_to_lds_m0(res, voff, soff);
        }
    };
    // next K tile: the two bases advance inside their resource words (two scalar instructions each; the bases are
    // 48-bit addresses, so the carry into word 1 stays inside its address field)
    auto advance_base = [](int4v& res, long step) {
        const uint64_t b = (((uint64_t)(uint32_t)res[1] << 32) | (uint32_t)res[0]) + (uint64_t)step;
        res[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)b);
        res[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    };
    auto advance_copies = [&]() {
        advance_base(a_res, a_k_step);
        advance_base(b_res, b_k_step);
    };
    auto issue_copies = [&](auto sc) {
        static_for<0, NCOPY>([&](auto dc) { issue_copy(sc, dc, std::integral_constant<int, 0>{}); });
        advance_copies();
    };
    // The MFMA is issued with the B fragment as first operand, i.e. it produces the transposed block: lane l ends up
    // with C[m = l % 16][n = 4 (l / 16) .. +3] of the block, 4 consecutive columns of one row.
    // one substep: the MFMAs on (afc, bfc); in slot m, `hook(m)` issues what rides along
    auto substep = [&](const V8(&afc)[TM], const V8(&bfc)[TN], auto&& hook) {
        static_for<0, NSLOT>([&](auto mc) {
            constexpr int m = decltype(mc)::value;
            // boustrophedon order over the wave's blocks: from one MFMA to the next exactly one of the two operand
            // fragments changes (at the end of a row of blocks the B fragment stays and A moves on), which costs less
            // switching energy than changing both; on this power-limited part that is worth 1-1.5 % at 8192^3
            constexpr int i = m / TN, j = (i & 1) ? TN - 1 - m % TN : m % TN;
            acc[i][j] = Elem<T>::mfma16(bfc[j], afc[i], acc[i][j]);
            hook(mc);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // the fragment reads that ride in slot m: fragments m, m + NSLOT, .. (a wave with a single row or column of blocks has
    // more fragments than MFMAs per substep)
    auto frags_of_slot = [&](auto sc, auto kc, auto mc, V8(&afn)[TM], V8(&bfn)[TN]) {
        constexpr int m = decltype(mc)::value;
        if constexpr (m < NFRAG) load_frag(sc, kc, mc, afn, bfn);
        if constexpr (m + NSLOT < NFRAG) load_frag(sc, kc, std::integral_constant<int, m + NSLOT>{}, afn, bfn);
        static_assert(NFRAG <= 2 * NSLOT, "at most two fragment reads per slot");
    };
    // copy d of a tile goes out in slot d * kCopySpacing of the substep behind the barrier that frees its stage: every
    // second slot where there are that many (buffer loads are cheap to issue in a row, and the earlier a copy leaves the
    // more time it has to land), evenly over the substep otherwise
    constexpr int kCopySpacingNum = NSLOT >= 2 * NCOPY ? 8 : 4 * NSLOT / NCOPY, kCopySpacingDen = 4;
    static_assert((NCOPY - 1) * kCopySpacingNum / kCopySpacingDen < NSLOT, "copies go out within one substep");
    // where a substep has a slot to spare, M0 is set one slot ahead of its load
    constexpr bool kSplitM0 = (NCOPY - 1) * kCopySpacingNum / kCopySpacingDen + 1 < NSLOT;
    auto copies_of_slot = [&](auto sc, auto gc) {   // issue the copies whose slot is g
        constexpr int g = decltype(gc)::value;
        static_for<0, NCOPY>([&](auto dc) {
            constexpr int slot = decltype(dc)::value * kCopySpacingNum / kCopySpacingDen;
            if constexpr (!kSplitM0) {
                if constexpr (slot == g) issue_copy(sc, dc, std::integral_constant<int, 0>{});
            } else {
                if constexpr (slot + 1 == g) issue_copy(sc, dc, std::integral_constant<int, 2>{});
            }
        });
        if constexpr (kSplitM0)
            static_for<0, NCOPY>([&](auto dc) {
                if constexpr (decltype(dc)::value * kCopySpacingNum / kCopySpacingDen == g) issue_copy(sc, dc, std::integral_constant<int, 1>{});
            });
    };
    // Ring of NSTAGE stages, tile t in stage t % NSTAGE. The prologue fills every stage; in tile kt, behind the barrier,
    // the copies of tile kt + NSTAGE go into the stage tile kt has just left. At that barrier tile kt+1 must have
    // landed: all but the copies of the NSTAGE-2 tiles issued after it.
    constexpr int NSTAGE = Cfg::NSTAGE;
    V8 af[2][TM], bf[2][TN];
    using Sub0 = std::integral_constant<int, 0>;
    using Sub1 = std::integral_constant<int, 1>;
    // The first tile is the one at the end of K. Its copies fetch nothing for k >= K: such a lane's offset is moved out
    // of the range of the resource (2 GiB for these copies; offsets inside a tile stay below that), and a copy that is
    // out of range writes zeros to LDS. Then the bases go back to k = 0 (with K a multiple of 64 the first tile is the
    // one at k = 0 and the bases move on to the next: the tiles are then walked in memory order).
    {
        constexpr uint32_t kOutOfRange = 0x80000000u;   // with any uniform offset added it stays at or above the range, without wrapping
        a_res[2] = (int)0x80000000u;
        b_res[2] = (int)0x80000000u;
        static_for<0, NCOPY>([&](auto dc) {
            constexpr int d = decltype(dc)::value;
            constexpr bool is_a = d < Cfg::A_INSTS;
            constexpr int e = is_a ? d : d - Cfg::A_INSTS;
            constexpr int dst = is_a ? e * Cfg::NWAVES * 1024 : kBRegion + e * Cfg::NWAVES * 1024;
            uint32_t voff, soff = 0u;
            if constexpr (RAGGED && is_a) voff = a_voff[e];
            else if constexpr (RAGGED) voff = b_voff[e];
            else { voff = is_a ? a_lane_off : b_lane_off; soff = e * (is_a ? a_copy_step : b_copy_step); }
            int k_of_lane;   // first k (inside the tile) of the 16 bytes this lane copies
            if constexpr (is_a ? A_KC : B_KC) {
                using TK = std::conditional_t<is_a, ATK, BTK>;
                const int row = wave * TK::kRowsPerInst + lane / TK::kChunksPerRow;
                k_of_lane = ((lane % TK::kChunksPerRow) ^ TK::swz(row)) * 8;
            } else {
                using TC = std::conditional_t<is_a, ATM, BTN>;
                k_of_lane = wave * TC::kRowsPerInst + lane / TC::kChunksPerRow + e * TC::kRowsPerPass;
            }
            if (k_of_lane >= k_first) voff = kOutOfRange;
            copy16_buffer_to_lds_at<dst>(is_a ? a_res : b_res, voff, soff, wave_lds);
        });
        advance_base(a_res, k_first < BK ? -first_tile * a_k_step : a_k_step);
        advance_base(b_res, k_first < BK ? -first_tile * b_k_step : b_k_step);
    }
    static_for<1, NSTAGE>([&](auto sc) {
        const int records = sign_mask_scalar(decltype(sc)::value - ktiles);
        a_res[2] = records;
        b_res[2] = records;
        issue_copies(sc);
    });
    wait_vmcnt<NCOPY * (NSTAGE - 1)>();
    __syncthreads();
    load_frags(Sub0{}, Sub0{}, af[0], bf[0]);

    // One K tile in stage sc (a compile-time constant: the loop below is unrolled over the ring). Every tile issues the
    // same instructions, so the count the waits rely on never changes: once no tile is left to fetch, the copies run on
    // an empty buffer (num_records = 0: out of range, nothing is fetched).
    auto tile = [&](auto sc, int kt) {
        using Next = std::integral_constant<int, (decltype(sc)::value + 1) % NSTAGE>;
        substep(af[0], bf[0], [&](auto mc) { frags_of_slot(sc, Sub1{}, mc, af[1], bf[1]); });
        // my copies of the next tile have landed and my reads of this stage are complete; after the barrier that holds
        // for every wave, so this stage may be refilled and the next one may be read
        wait_vmcnt<NCOPY * (NSTAGE - 2)>();
        __syncthreads();
        const int records = sign_mask_scalar(kt + NSTAGE - ktiles);   // -1 while a tile is left to fetch, else 0
        a_res[2] = records;
        b_res[2] = records;
        substep(af[1], bf[1], [&](auto mc) {
            frags_of_slot(Next{}, Sub0{}, mc, af[0], bf[0]);
            copies_of_slot(sc, mc);   // tile kt + NSTAGE
        });
        advance_copies();
    };
    int kt = 0;
    MI355_TL(tl_w[1] = timeline::wall_clock(); tl_c[0] = timeline::shader_cycles();)
    for (; kt < ktiles; kt += NSTAGE)
        static_for<0, NSTAGE>([&](auto sc) {
            if (kt + decltype(sc)::value < ktiles) tile(sc, kt + decltype(sc)::value);
        });
    MI355_TL(tl_w[2] = timeline::wall_clock(); tl_c[1] = timeline::shader_cycles();)

    // ---- epilogue ------------------------------------------------------------------------------------------------
    constexpr int TNO = EPI == 1 ? TN / 2 : TN;   // column blocks a wave stores
    static_assert(Cfg::NWAVES * TM * 16 * TNO * 32 <= Cfg::LDS_BYTES, "epilogue staging does not fit in LDS");
    wait_vmcnt<0>();  // the last tiles' copies (on the empty buffer) have written their zeros
    __syncthreads();  // every wave has finished reading the operand stages
    if constexpr (SPLIT_K) {
        // partial tile (block, range): element q of lane t's accumulator block b at float (b * 4 + q) * NTHREADS + t, so
        // that every store and load instruction of a wave covers 256 contiguous bytes
        const long tile_floats = (long)Cfg::NTHREADS * TM * TN * 4;
        float* tile_part = part + (long)blockIdx.x * splits * tile_floats;
        float* mine = tile_part + (long)blockIdx.y * tile_floats + tid;
        // (device-scope atomic stores, i.e. `global_store_dword .. sc1`, written as such so that the compiler places the
        // wait states between the last matrix instructions and the first memory instruction that reads their result: a
        // wave that arrives last at the barrier above is only a few cycles behind its last MFMA)
#pragma unroll
        for (int b = 0; b < TM * TN; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                __hip_atomic_store(mine + (long)(b * 4 + q) * Cfg::NTHREADS, acc[b / TN][b % TN][q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this lane's part has reached memory before the ticket is drawn
        __syncthreads();
        MI355_LDS unsigned* ticket_sh = (MI355_LDS unsigned*)smem;
        if (tid == 0) *ticket_sh = __hip_atomic_fetch_add(&counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const unsigned ticket = *ticket_sh;
        __syncthreads();   // the epilogue below reuses that LDS
        if (ticket != (unsigned)(splits - 1)) return;
        // the last one: every other workgroup of this tile drew its ticket after its part had reached memory. The parts
        // are read with device-coherent loads (sc1), 16 in flight per lane, and added in the order of the ranges.
#pragma unroll
        for (int b = 0; b < TM * TN; ++b) {
            float4v sum = float4v{0.f, 0.f, 0.f, 0.f};
            for (int r0 = 0; r0 < splits; r0 += 4) {
                float4v v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const float* pa = tile_part + (long)min(r0 + u, splits - 1) * tile_floats + (long)(b * 4) * Cfg::NTHREADS + tid;
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        asm volatile("global_load_dword %0, %1, off sc1" : "=v"(v[u][q]) : "v"(pa + (long)q * Cfg::NTHREADS) : "memory");
                }
                asm volatile("s_waitcnt vmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) :: "memory");
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (r0 + u < splits) sum += v[u];
            }
            acc[b / TN][b % TN] = sum;
        }
        if (tid == 0) __hip_atomic_store(&counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    store_wave_tile<T, TM, TN, EPI, RAGGED>(acc, smem + wave * (TM * 16 * TNO * 32), C, R, m0 + wm * TM * 16,
                                            (EPI == 1 ? n0 / 2 : n0) + wn * TNO * 16, M, EPI == 1 ? N / 2 : N, ldc, ldr, lane);
    MI355_TL(
        wait_vmcnt<0>();   // the stores of this wave have been accepted
        tl_w[3] = timeline::wall_clock();
        if (tid == 0 && blockIdx.x < timeline::kMaxWorkgroups) {
            unsigned long long* rec = hgemm_stamps + (long)blockIdx.x * timeline::kSlots;
            rec[0] = tl_w[0]; rec[1] = tl_w[1]; rec[2] = tl_w[2]; rec[3] = tl_w[3];
            rec[4] = tl_c[0]; rec[5] = tl_c[1]; rec[6] = (unsigned long long)ktiles; rec[7] = 0;
        })
}

// ---------------------------------------------------------------------------------------------------------
// Bounds-checked kernel for any shape: 64x64 tile per wave-quad, operands gathered with guarded scalar loads
// into the MFMA layout. Used for shapes the tiled kernels do not cover; correctness first.
// ---------------------------------------------------------------------------------------------------------
template <typename T, bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void hgemm_edge_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                         T* C, const T* R, int M, int N, int K, long lda,
                                                         long ldb, long ldc, long ldr) {
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    using V2 = typename Elem<T>::v2;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const long m = (long)blockIdx.y * 64 + (wave >> 1) * 32 + (lane & 31);
    const long n = (long)blockIdx.x * 64 + (wave & 1) * 32 + (lane & 31);
    const int kh = 8 * (lane >> 5);
    float16v acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
        V8 a, b;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            int k = k0 + kh + j;
            bool kin = k < K;
            T av = (T)0.f, bv = (T)0.f;
            if (kin && m < M) av = A_KC ? A[m * lda + k] : A[(long)k * lda + m];
            if (kin && n < N) bv = B_KC ? B[n * ldb + k] : B[(long)k * ldb + n];
            a[j] = av;
            b[j] = bv;
        }
        acc = Elem<T>::mfma32(a, b, acc);
    }
    // acc element 4p+q is C[row 8p + 4*(lane/32) + q][col lane%32] of this wave's 32x32 block
    const long rb = (long)blockIdx.y * 64 + (wave >> 1) * 32 + 4 * (lane >> 5);
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            long r = rb + 8 * p + q;
            if (r < M && n < N) {
                T v = (T)acc[4 * p + q];
                if (R != nullptr) v = (T)((float)v + (float)R[r * ldr + n]);
                C[r * ldc + n] = v;
            }
        }
}

// ---------------------------------------------------------------------------------------------------------
// Small-M kernel (decode-shaped GEMM, M <= 16 rows per workgroup row), layouts NN and TN. HBM-bound: B is streamed once.
//   * a workgroup owns 64 columns of C; its 8 waves split K between them (in-workgroup split-K, reduced
//     through LDS at the end, so no global workspace and no atomics);
//   * every wave runs its own copy pipeline, without workgroup barriers: per 32-deep k-step it copies a
//     32x64 slab of B (4 KiB) and a 16x32 slab of A (1 KiB) global -> LDS with 16-byte direct-to-LDS copies,
//     keeps kSmallMStages-1 steps in flight, and waits for the oldest with s_waitcnt vmcnt;
//   * B fragments are read with the transposing LDS read, the product is MFMA 16x16x32;
//   * layout TN (A stored [K,M], A_KC = false): the A slab of a k-step is 32 rows (k) x 16 m, copied as it lies and read
//     with the transposing read like B. Its 16-byte chunks hold 8 rows of the product: the chunks of the rows M .. M
//     rounded up to 8 lie in the padding of A's rows (lda is a multiple of 8 and at least M), their rows of the product
//     are never stored; chunks past that fold back onto the last one.
// ---------------------------------------------------------------------------------------------------------
constexpr int kSmallMWaves = 8;
constexpr int kSmallMStages = 3;
constexpr int kSmallMStageBytes = 5 * 1024;  // 4 KiB of B + 1 KiB of A
constexpr int kSmallMWaveBytes = kSmallMStages * kSmallMStageBytes;
constexpr int kSmallMLdsBytes = kSmallMWaves * kSmallMWaveBytes;
static_assert(kSmallMLdsBytes >= kSmallMWaves * 1024 * 4, "the reduction reuses the pipeline memory");

template <typename T, bool A_KC>
__global__ __launch_bounds__(kSmallMWaves * 64) void hgemm_smallm_nn_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                              T* C, const T* R, int M, int N, int K, long lda,
                                                              long ldb, long ldc, long ldr, int n_tiles) {
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    using V2 = typename Elem<T>::v2;
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Workgroup i takes column tile i: neighbouring tiles (the 128-byte pieces of one row of B) then run at the same time on
    // different XCDs. Keeping them on one XCD (tile = (i % 8) * (n_tiles / 8) + i / 8) was 3-5 % slower, cached or not
    // (16 x 14336 x 4096: 20.2 -> 19.2 us on a re-read weight, 26.4 -> 25.6 us on one that comes from HBM).
    const int tile = blockIdx.x;
    const int n0 = tile * 64;
    const int m0 = blockIdx.y * 16;

    const int ksteps = K / 32;
    const int s_begin = (int)((long)wave * ksteps / kSmallMWaves);
    const int s_end = (int)((long)(wave + 1) * ksteps / kSmallMWaves);

    MI355_LDS char* wbase = smem + wave * kSmallMWaveBytes;

    // ---- copy descriptors -------------------------------------------------------------------------------
    // B slab: 32 rows (k) x 128 bytes; copy i covers rows 8i .. 8i+7, chunk position lane%8, chunk c of row r
    // is stored at position c ^ 2*(r%4) (keeps the 16 lanes of a transposing read on distinct banks)
    const int b_row = lane >> 3;                                  // + 8*i
    const int b_chunk = (lane & 7) ^ (2 * (b_row & 3));           // (8i + b_row) % 4 == b_row % 4
    const int n_chunk_max = N / 8 - 1;
    const int b_col = min(n0 / 8 + b_chunk, n_chunk_max) * 8;     // clamp: columns past N are never stored
    const T* b_src = B + (long)(s_begin * 32 + b_row) * ldb + b_col;
    // A slab: 16 rows (m) x 64 bytes; row lane/4, chunk position lane%4, chunk c of row r at c ^ ((r>>1)&3)
    // A stored [K,M]: slab of 32 rows (k) x 32 bytes; LDS row slot lane/2 holds k row = slot with bits 2 and 3 swapped,
    // which puts the 8 rows that lanes 0..31 of a transposing read touch (k 0..3 and 8..11, + 4 for the second read)
    // into 8 consecutive slots = 256 bytes = distinct banks. Chunks past M fold back onto the last 8 rows of A.
    const int a_row = lane >> 2;
    const int a_chunk = (lane & 3) ^ ((a_row >> 1) & 3);
    const int at_slot = lane >> 1;
    const int at_k = (at_slot & ~12) | ((at_slot & 4) << 1) | ((at_slot & 8) >> 1);
    const T* a_src = A_KC ? A + (long)min(m0 + a_row, M - 1) * lda + (long)s_begin * 32 + a_chunk * 8
                          : A + (long)(s_begin * 32 + at_k) * lda + min(m0 + 8 * (lane & 1), ((M + 7) & ~7) - 8);

    auto issue_stage = [&](int slot) {
        MI355_LDS char* st = wbase + slot * kSmallMStageBytes;
#pragma unroll
        for (int i = 0; i < 4; ++i) copy16_global_to_lds(b_src + (long)(8 * i) * ldb, st + i * 1024);
        copy16_global_to_lds(a_src, st + 4096);
        b_src += 32 * ldb;
        a_src += A_KC ? 32 : 32 * lda;
    };

    // ---- fragment read offsets inside a stage ---------------------------------------------------------------
    // A fragment: lane holds A[m = lane%16][k = 8*(lane/16) .. +7]
    // (A stored [K,M]: transposing read of k rows 8*(lane/16) + 4t + (lane%16)/4, m = 4*(lane%4) .. +3; the second read
    //  (t = 1, k + 4) lies 8 slots = 256 bytes further)
    const int at_read_k = 8 * (lane >> 4) + ((lane & 15) >> 2);
    const int at_read_slot = (at_read_k & ~12) | ((at_read_k & 4) << 1) | ((at_read_k & 8) >> 1);
    const int a_off = A_KC ? 4096 + (lane & 15) * 64 + (((lane >> 4) ^ (((lane & 15) >> 1) & 3)) << 4)
                           : 4096 + at_read_slot * 32 + (lane & 3) * 8;
    // B fragment of column block j: rows 8*(lane/16) + 4t + (lane%16)/4, columns 16j + 4*(lane%4) .. +3
    const int bt_row = 8 * (lane >> 4) + ((lane & 15) >> 2);
    const int bt_swz = 2 * (bt_row & 3);
    int b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int chunk = (2 * j + ((lane & 3) >> 1)) ^ bt_swz;
        b_off[j] = bt_row * 128 + chunk * 16 + (lane & 1) * 8;
    }

    float4v acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[j] = float4v{0.f, 0.f, 0.f, 0.f};

    // ---- pipeline ---------------------------------------------------------------------------------------------
    int issued = s_begin;
#pragma unroll
    for (int i = 0; i < kSmallMStages - 1; ++i)
        if (issued < s_end) {
            issue_stage(i);
            ++issued;
        }
    int slot = 0, fill = kSmallMStages - 1;
    for (int s = s_begin; s < s_end; ++s) {
        if (issued < s_end) {
            issue_stage(fill);
            ++issued;
            fill = (fill + 1 == kSmallMStages) ? 0 : fill + 1;
            wait_vmcnt<5 * (kSmallMStages - 1)>();  // everything but the newest kSmallMStages-1 steps has landed
        } else {
            wait_vmcnt<0>();
        }
        MI355_LDS char* st = wbase + slot * kSmallMStageBytes;
        slot = (slot + 1 == kSmallMStages) ? 0 : slot + 1;
        V8 af;
        if constexpr (A_KC) af = Elem<T>::frag(lds_read_b128(st + a_off));
        else af = Elem<T>::frag(concat(lds_read_tr16_b64(st + a_off), lds_read_tr16_b64(st + a_off + 256)));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            half4 lo = lds_read_tr16_b64(st + b_off[j]);
            half4 hi = lds_read_tr16_b64(st + b_off[j] + 4 * 128);
            acc[j] = Elem<T>::mfma16(af, Elem<T>::frag(concat(lo, hi)), acc[j]);
        }
        // the reads of this slot must be complete before a later copy refills it
        wait_lgkmcnt<0>();
    }

    // ---- reduce the 8 partial tiles through LDS ---------------------------------------------------------------
    // acc[j][q] is D[m = 4*(lane/16) + q][n = 16j + lane%16]
    __syncthreads();  // every wave is done with its staging memory
    MI355_LDS float* red = (MI355_LDS float*)smem;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) red[wave * 1024 + (4 * (lane >> 4) + q) * 64 + 16 * j + (lane & 15)] = acc[j][q];
    __syncthreads();
    for (int o = tid * 2; o < 1024; o += kSmallMWaves * 128) {  // two neighbouring columns of one row
        float s0 = 0.f, s1 = 0.f;
#pragma unroll
        for (int w = 0; w < kSmallMWaves; ++w) {
            s0 += red[w * 1024 + o];
            s1 += red[w * 1024 + o + 1];
        }
        const int m = m0 + (o >> 6);
        const int n = n0 + (o & 63);
        if (m < M && n < N) {
            V2 v;
            v[0] = (T)s0;
            v[1] = (T)s1;
            if (R != nullptr) {
                const V2 r = *(const V2*)(R + (long)m * ldr + n);
                v[0] = (T)((float)v[0] + (float)r[0]);
                v[1] = (T)((float)v[1] + (float)r[1]);
            }
            *(V2*)(C + (long)m * ldc + n) = v;
        }
    }
}

template <typename T, bool A_KC>
static hipError_t launch_smallm_nn(const T* A, const T* B, T* C, const T* R, int M, int N, int K, long lda, long ldb,
                                   long ldc, long ldr, hipStream_t stream) {
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(hgemm_smallm_nn_kernel<T, A_KC>), kSmallMLdsBytes); e != hipSuccess) return e;
    const int n_tiles = (N + 63) / 64;
    dim3 grid(n_tiles, (M + 15) / 16);
    hgemm_smallm_nn_kernel<T, A_KC><<<grid, dim3(kSmallMWaves * 64), kSmallMLdsBytes, stream>>>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, n_tiles);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// Small-M kernel for layout NT (B stored [N,K]: the nn.Linear weight layout of decode-time projections), M <= 16
// rows per workgroup row. HBM-bound like hgemm_smallm_nn_kernel and built the same way: a workgroup owns 16
// columns of C (16 rows of B), its waves split K and are reduced through LDS; every wave runs a private,
// barrier-free copy pipeline of 64-deep k-steps (16x64 of B and 16x64 of A, 2 KiB each, direct-to-LDS), both
// operands are K-contiguous so both fragments are plain ds_read_b128, the product is MFMA 16x16x32.
// Four waves with four stages each = 64 KiB of LDS, so that two or three workgroups share a CU and one's start-up
// and reduction hide under the others' streaming: with weights that come from HBM (not from the memory-side cache, as
// when one weight matrix is launched on again and again) that beats eight waves on 128 KiB, one workgroup per CU, by
// 7-15 % (8 x 4096 x 14336: 21.7 us against 23.3, 8 x 6144 x 4096: 11.9 against 13.4).
// ---------------------------------------------------------------------------------------------------------
constexpr int kSmallMNtWaves = 4;
constexpr int kSmallMNtStages = 4;
constexpr int kSmallMNtStageBytes = 4 * 1024;  // 2 KiB of B + 2 KiB of A
constexpr int kSmallMNtWaveBytes = kSmallMNtStages * kSmallMNtStageBytes;
constexpr int kSmallMNtLdsBytes = kSmallMNtWaves * kSmallMNtWaveBytes;
static_assert(kSmallMNtLdsBytes >= kSmallMNtWaves * 256 * 4, "the reduction reuses the pipeline memory");

// GATE_UP: the rows of B come in groups of [32 gate | 32 up] (the operand of the tiled kernels' gate/up epilogue) and C is
// silu(gate) * up, half as wide. Workgroup t then takes the 8 gate rows 64 (t / 4) + 8 (t % 4) .. +7 and the 8 up rows 32
// further on, and stores the 8 columns 32 (t / 4) + 8 (t % 4) .. +7 of C.
template <typename T, bool HALF_A, bool GATE_UP>
__global__ __launch_bounds__(kSmallMNtWaves * 64) void hgemm_smallm_nt_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                              T* C, const T* R, int M, int N, int K, long lda,
                                                              long ldb, long ldc, long ldr, int n_tiles) {
    using V8 = typename Elem<T>::v8;
    using V4 = typename Elem<T>::v4;
    using V2 = typename Elem<T>::v2;
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    int tile = blockIdx.x;
    if (n_tiles % 8 == 0) tile = (blockIdx.x % 8) * (n_tiles / 8) + blockIdx.x / 8;
    const int n0 = tile * 16;
    const int m0 = blockIdx.y * 16;

    const int ksteps = K / 64;
    const int s_begin = (int)((long)wave * ksteps / kSmallMNtWaves);
    const int s_end = (int)((long)(wave + 1) * ksteps / kSmallMNtWaves);
    MI355_LDS char* wbase = smem + wave * kSmallMNtWaveBytes;

    // slab = 16 rows x 128 bytes; a copy instruction covers 8 rows (row lane/8, chunk position lane%8);
    // chunk c of row r is stored at position c ^ (r & 7)
    const int c_row = lane >> 3;  // + 8*i
    const int c_chunk = (lane & 7) ^ (c_row & 7);
    const int b_row0 = GATE_UP ? 64 * (tile >> 2) + 8 * (tile & 3) + c_row : n0 + c_row;
    const int b_row1 = GATE_UP ? b_row0 + 32 : b_row0 + 8;
    const T* b_src0 = B + (long)min(b_row0, N - 1) * ldb + (long)s_begin * 64 + c_chunk * 8;
    const T* b_src1 = B + (long)min(b_row1, N - 1) * ldb + (long)s_begin * 64 + c_chunk * 8;
    const T* a_src0 = A + (long)min(m0 + c_row, M - 1) * lda + (long)s_begin * 64 + c_chunk * 8;
    const T* a_src1 = A + (long)min(m0 + c_row + 8, M - 1) * lda + (long)s_begin * 64 + c_chunk * 8;

    // HALF_A (M <= 8): rows 8..15 of the A slab are not copied; the fragment rows read from there hold whatever the
    // memory held, and so do rows 8..15 of the product, which are never stored (an output row depends on its own A row only)
    constexpr int kCopies = HALF_A ? 3 : 4;
    auto issue_stage = [&](int slot) {
        MI355_LDS char* st = wbase + slot * kSmallMNtStageBytes;
        copy16_global_to_lds(b_src0, st);
        copy16_global_to_lds(b_src1, st + 1024);
        copy16_global_to_lds(a_src0, st + 2048);
        if constexpr (!HALF_A) copy16_global_to_lds(a_src1, st + 3072);
        b_src0 += 64;
        b_src1 += 64;
        a_src0 += 64;
        a_src1 += 64;
    };

    // fragment of k-substep sub (32 deep): lane holds X[row = lane%16][k = 32*sub + 8*(lane/16) .. +7]
    const int f_row = lane & 15;
    int f_off[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) f_off[sub] = f_row * 128 + (((4 * sub + (lane >> 4)) ^ (f_row & 7)) << 4);

    float4v acc = float4v{0.f, 0.f, 0.f, 0.f};

    int issued = s_begin;
#pragma unroll
    for (int i = 0; i < kSmallMNtStages - 1; ++i)
        if (issued < s_end) {
            issue_stage(i);
            ++issued;
        }
    int slot = 0, fill = kSmallMNtStages - 1;
    for (int s = s_begin; s < s_end; ++s) {
        if (issued < s_end) {
            issue_stage(fill);
            ++issued;
            fill = (fill + 1 == kSmallMNtStages) ? 0 : fill + 1;
            wait_vmcnt<kCopies * (kSmallMNtStages - 1)>();  // everything but the newest kSmallMNtStages-1 steps has landed
        } else {
            wait_vmcnt<0>();
        }
        MI355_LDS char* st = wbase + slot * kSmallMNtStageBytes;
        slot = (slot + 1 == kSmallMNtStages) ? 0 : slot + 1;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            V8 bf = Elem<T>::frag(lds_read_b128(st + f_off[sub]));
            V8 af = Elem<T>::frag(lds_read_b128(st + 2048 + f_off[sub]));
            acc = Elem<T>::mfma16(af, bf, acc);
        }
        wait_lgkmcnt<0>();  // the reads of this slot are complete before a later copy refills it
    }

    // acc[q] is D[m = 4*(lane/16) + q][n = lane%16]; reduce the 8 partial tiles through LDS
    __syncthreads();
    MI355_LDS float* red = (MI355_LDS float*)smem;
#pragma unroll
    for (int q = 0; q < 4; ++q) red[wave * 256 + (4 * (lane >> 4) + q) * 16 + (lane & 15)] = acc[q];
    __syncthreads();
    for (int o = tid; o < 256; o += kSmallMNtWaves * 64) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < kSmallMNtWaves; ++w) sum += red[w * 256 + o];
        const int m = m0 + (o >> 4);
        if constexpr (GATE_UP) {
            if ((o & 15) < 8 && m < M) {   // column o % 16 is a gate, the one 8 further on its up
                float up = 0.f;
#pragma unroll
                for (int w = 0; w < kSmallMNtWaves; ++w) up += red[w * 256 + o + 8];
                const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-sum * 1.4426950408889634f));
                C[(long)m * ldc + 32 * (tile >> 2) + 8 * (tile & 3) + (o & 15)] = (T)(sum * sig * up);
            }
            continue;
        }
        const int n = n0 + (o & 15);
        if (m < M && n < N) {
            T v = (T)sum;
            if (R != nullptr) v = (T)((float)v + (float)R[(long)m * ldr + n]);
            C[(long)m * ldc + n] = v;
        }
    }
}

// The same product for wide weights (at least a few hundred row tiles) and K = 256 STEPS: a workgroup takes TPW
// consecutive row tiles and keeps its slice of A in registers after the first of them (a wave's K / 4 columns of the 16
// rows: 2 STEPS fragments, 128 registers at K = 4096), so from the second tile on only the weights are copied: the
// activation rows are then fetched from L2 once per TPW tiles instead of once per tile (they are as many bytes through
// the CU's memory pipeline as the weights themselves). The stream over (tile, k-step) is unrolled completely: every LDS
// offset, copy destination and wait count is an immediate, a k-step is ~18 instructions. The partial
// tiles of the four waves meet in LDS once, behind the stream (no barrier inside it).
template <typename T, bool HALF_A, bool GATE_UP, int STEPS, int TPW>
__global__ __launch_bounds__(kSmallMNtWaves * 64) void hgemm_smallm_nt_rega_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                                   T* C, const T* R, int M, int N, long lda, long ldb,
                                                                   long ldc, long ldr, int n_groups) {
    using V8 = typename Elem<T>::v8;
    constexpr int NST = kSmallMNtStages, TOTAL = TPW * STEPS;
    constexpr int kCopiesA = HALF_A ? 1 : 2;
    extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
    MI355_LDS char* smem = (MI355_LDS char*)smem_raw;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    int group = blockIdx.x;
    if (n_groups % 8 == 0) group = (blockIdx.x % 8) * (n_groups / 8) + blockIdx.x / 8;
    const int tile0 = group * TPW;
    const long kbase = (long)wave * STEPS * 64;

    // slab = 16 rows x 128 bytes; a copy instruction covers 8 rows (row lane/8, chunk position lane%8); chunk c of row r is
    // stored at position c ^ (r & 7). Lane offsets are relative to the tile's first row and the wave's first column.
    const int c_row = lane >> 3;
    const int c_chunk = (lane & 7) ^ (c_row & 7);
    const uint32_t b_voff0 = (uint32_t)((long)c_row * ldb * 2 + c_chunk * 16);
    const uint32_t b_voff1 = (uint32_t)((long)(c_row + (GATE_UP ? 32 : 8)) * ldb * 2 + c_chunk * 16);
    const uint32_t a_voff0 = (uint32_t)((long)min(c_row, M - 1) * lda * 2 + c_chunk * 16);
    const uint32_t a_voff1 = (uint32_t)((long)min(c_row + 8, M - 1) * lda * 2 + c_chunk * 16);
    const T* a_base = A + kbase;
    // first weight row of tile t (GATE_UP: 8 gate rows there, their 8 up rows 32 further on)
    const T* b_base[TPW];
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
        const int t = tile0 + i;
        b_base[i] = B + (long)(GATE_UP ? 64 * (t >> 2) + 8 * (t & 3) : t * 16) * ldb + kbase;
    }
    const uint32_t wave_lds = (uint32_t)(uintptr_t)(smem + wave * kSmallMNtWaveBytes);

    // fragment of k-substep sub (32 deep): lane holds X[row = lane%16][k = 32*sub + 8*(lane/16) .. +7]
    const int f_row = lane & 15;
    MI355_LDS char* f_ptr[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
        f_ptr[sub] = smem + wave * kSmallMNtWaveBytes + f_row * 128 + (((4 * sub + (lane >> 4)) ^ (f_row & 7)) << 4);
    MI355_LDS float* red = (MI355_LDS float*)(smem + kSmallMNtLdsBytes);   // [TPW][waves][256]

    V8 areg[STEPS][2];
    float4v acc = float4v{0.f, 0.f, 0.f, 0.f};

    auto copies_of = [](int u) { return u >= TOTAL ? 0 : u < STEPS ? 2 + kCopiesA : 2; };
    auto issue = [&](auto uc) {
        constexpr int u = decltype(uc)::value, i = u / STEPS, st = u % STEPS, slot = u % NST;
        const T* bb = b_base[i] + st * 64;   // scalar pointer arithmetic
        copy16_global_to_lds_imm<slot * kSmallMNtStageBytes>(bb, b_voff0, wave_lds);
        copy16_global_to_lds_imm<slot * kSmallMNtStageBytes + 1024>(bb, b_voff1, wave_lds);
        if constexpr (i == 0) {
            const T* ab = a_base + st * 64;
            copy16_global_to_lds_imm<slot * kSmallMNtStageBytes + 2048>(ab, a_voff0, wave_lds);
            if constexpr (!HALF_A) copy16_global_to_lds_imm<slot * kSmallMNtStageBytes + 3072>(ab, a_voff1, wave_lds);
        }
    };
    static_for<0, NST - 1>([&](auto uc) { issue(uc); });
    static_for<0, TOTAL>([&](auto uc) {
        constexpr int u = decltype(uc)::value, i = u / STEPS, st = u % STEPS, slot = u % NST;
        if constexpr (u + NST - 1 < TOTAL) issue(std::integral_constant<int, u + NST - 1>{});
        wait_vmcnt<copies_of(u + 1) + copies_of(u + 2) + copies_of(u + 3)>();   // everything up to step u has landed
        static_assert(NST == 4, "the wait above counts the three steps in flight behind step u");
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            V8 bf = Elem<T>::frag(lds_read_b128(f_ptr[sub] + slot * kSmallMNtStageBytes));
            if constexpr (i == 0) areg[st][sub] = Elem<T>::frag(lds_read_b128(f_ptr[sub] + (slot * kSmallMNtStageBytes + 2048)));
            acc = Elem<T>::mfma16(areg[st][sub], bf, acc);
        }
        wait_lgkmcnt<0>();  // the reads of this slot are complete before a later copy refills it
        if constexpr (st == STEPS - 1) {   // acc[q] is D[m = 4*(lane/16) + q][n = lane%16] of tile i
#pragma unroll
            for (int q = 0; q < 4; ++q) red[(i * kSmallMNtWaves + wave) * 256 + (4 * (lane >> 4) + q) * 16 + (lane & 15)] = acc[q];
            acc = float4v{0.f, 0.f, 0.f, 0.f};
        }
    });

    __syncthreads();
    for (int o = tid; o < TPW * 256; o += kSmallMNtWaves * 64) {
        const int i = o >> 8, e = o & 255, tile = tile0 + i;
        const MI355_LDS float* rt = red + i * kSmallMNtWaves * 256;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < kSmallMNtWaves; ++w) sum += rt[w * 256 + e];
        const int m = e >> 4;
        if constexpr (GATE_UP) {
            if ((e & 15) < 8 && m < M) {   // column e % 16 is a gate, the one 8 further on its up
                float up = 0.f;
#pragma unroll
                for (int w = 0; w < kSmallMNtWaves; ++w) up += rt[w * 256 + e + 8];
                const float sig = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-sum * 1.4426950408889634f));
                C[(long)m * ldc + 32 * (tile >> 2) + 8 * (tile & 3) + (e & 15)] = (T)(sum * sig * up);
            }
        } else {
            const int n = tile * 16 + (e & 15);
            if (m < M && n < N) {
                T v = (T)sum;
                if (R != nullptr) v = (T)((float)v + (float)R[(long)m * ldr + n]);
                C[(long)m * ldc + n] = v;
            }
        }
    }
}

// Tiles per workgroup for the kernel above, or 0 when it does not apply: K = 4096, at most 16 rows, whole tiles, and at
// least 192 workgroups left to keep the memory system busy. Measured on weights that come from HBM (a different weight
// matrix on every launch), against one tile per workgroup: 16 x 14336 x 4096 24.5 -> 21.7 us with four tiles (22.1 with
// two), 16 x 6144 x 4096 13.1 -> 11.4 (two), 16 x 28672 x 4096 43.2 -> 40.5 (four; 42.2 with two). Up to 8 rows, where
// the activation slab is half as large to begin with: 8 x 14336 x 4096 22.3 -> 20.5 us with two tiles (21.2 with four),
// 8 x 28672 x 4096 39.1 -> 39.4-39.9 either way, so the widest products keep one tile per workgroup there.
static int smallm_nt_rega_tpw(int M, int n_tiles, int K, long lda, long ldb) {
    if (M > 16 || K != 4096 || lda >= (1L << 22) || ldb >= (1L << 22)) return 0;   // lane offsets of up to 40 rows in 32 bits
    if (M <= 8) return n_tiles % 2 == 0 && n_tiles / 2 >= 192 && n_tiles / 2 <= 512 ? 2 : 0;
    for (int tpw : {4, 2})
        if (n_tiles % tpw == 0 && n_tiles / tpw >= 192) return tpw;
    return 0;
}

template <typename T, bool HALF_A, bool GATE_UP>
static hipError_t launch_smallm_nt_rega(const T* A, const T* B, T* C, const T* R, int M, int N, long lda, long ldb, long ldc,
                                        long ldr, int n_tiles, int tpw, hipStream_t stream) {
    static DynamicLdsOnce once4, once2;
    const int groups = n_tiles / tpw;
    if (tpw == 4) {
        constexpr int lds = kSmallMNtLdsBytes + 4 * kSmallMNtWaves * 1024;
        auto kern = hgemm_smallm_nt_rega_kernel<T, HALF_A, GATE_UP, 16, 4>;
        if (hipError_t e = once4.ensure(reinterpret_cast<const void*>(kern), lds); e != hipSuccess) return e;
        kern<<<dim3(groups), dim3(kSmallMNtWaves * 64), lds, stream>>>(A, B, C, R, M, N, lda, ldb, ldc, ldr, groups);
    } else {
        constexpr int lds = kSmallMNtLdsBytes + 2 * kSmallMNtWaves * 1024;
        auto kern = hgemm_smallm_nt_rega_kernel<T, HALF_A, GATE_UP, 16, 2>;
        if (hipError_t e = once2.ensure(reinterpret_cast<const void*>(kern), lds); e != hipSuccess) return e;
        kern<<<dim3(groups), dim3(kSmallMNtWaves * 64), lds, stream>>>(A, B, C, R, M, N, lda, ldb, ldc, ldr, groups);
    }
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_smallm_nt(const T* A, const T* B, T* C, const T* R, int M, int N, int K, long lda, long ldb,
                                   long ldc, long ldr, hipStream_t stream) {
    static DynamicLdsOnce lds_once, lds_once_half;
    const int n_tiles = (N + 15) / 16;
    if (const int tpw = N % 16 == 0 ? smallm_nt_rega_tpw(M, n_tiles, K, lda, ldb) : 0; tpw > 0) {
        if (M <= 8) return launch_smallm_nt_rega<T, true, false>(A, B, C, R, M, N, lda, ldb, ldc, ldr, n_tiles, tpw, stream);
        return launch_smallm_nt_rega<T, false, false>(A, B, C, R, M, N, lda, ldb, ldc, ldr, n_tiles, tpw, stream);
    }
    dim3 grid(n_tiles, (M + 15) / 16);
    if (M <= 8) {
        if (hipError_t e = lds_once_half.ensure(reinterpret_cast<const void*>(hgemm_smallm_nt_kernel<T, true, false>), kSmallMNtLdsBytes); e != hipSuccess) return e;
        hgemm_smallm_nt_kernel<T, true, false><<<grid, dim3(kSmallMNtWaves * 64), kSmallMNtLdsBytes, stream>>>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, n_tiles);
    } else {
        if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(hgemm_smallm_nt_kernel<T, false, false>), kSmallMNtLdsBytes); e != hipSuccess) return e;
        hgemm_smallm_nt_kernel<T, false, false><<<grid, dim3(kSmallMNtWaves * 64), kSmallMNtLdsBytes, stream>>>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, n_tiles);
    }
    return hipGetLastError();
}

// silu(A gate^T) * (A up^T) for up to 16 rows: N counts the rows of B ([32 gate | 32 up] groups, a multiple of 64), C is
// [M, N / 2].
template <typename T>
static hipError_t launch_smallm_nt_gate_up(const T* A, const T* B, T* C, int M, int N, int K, long lda, long ldb, long ldc,
                                           hipStream_t stream) {
    static DynamicLdsOnce lds_once, lds_once_half;
    const int n_tiles = N / 16;
    if (const int tpw = smallm_nt_rega_tpw(M, n_tiles, K, lda, ldb); tpw > 0) {
        if (M <= 8) return launch_smallm_nt_rega<T, true, true>(A, B, C, nullptr, M, N, lda, ldb, ldc, 0, n_tiles, tpw, stream);
        return launch_smallm_nt_rega<T, false, true>(A, B, C, nullptr, M, N, lda, ldb, ldc, 0, n_tiles, tpw, stream);
    }
    dim3 grid(n_tiles, 1);
    if (M <= 8) {
        if (hipError_t e = lds_once_half.ensure(reinterpret_cast<const void*>(hgemm_smallm_nt_kernel<T, true, true>), kSmallMNtLdsBytes); e != hipSuccess) return e;
        hgemm_smallm_nt_kernel<T, true, true><<<grid, dim3(kSmallMNtWaves * 64), kSmallMNtLdsBytes, stream>>>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, n_tiles);
    } else {
        if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(hgemm_smallm_nt_kernel<T, false, true>), kSmallMNtLdsBytes); e != hipSuccess) return e;
        hgemm_smallm_nt_kernel<T, false, true><<<grid, dim3(kSmallMNtWaves * 64), kSmallMNtLdsBytes, stream>>>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, n_tiles);
    }
    return hipGetLastError();
}

template <typename T, bool A_KC, bool B_KC, int BM, int BN, int WM, int WN, int EPI = 0, bool RAGGED = false, int STAGES = 0, int PER_CU = 1>
static hipError_t launch_main(const T* A, const T* B, T* C, const T* R, int M, int N, int K, long lda, long ldb,
                              long ldc, long ldr, hipStream_t stream) {
    using Cfg = MainCfg<A_KC, B_KC, BM, BN, WM, WN, STAGES>;
    auto kern = hgemm_main_kernel<T, A_KC, B_KC, BM, BN, WM, WN, EPI, RAGGED, STAGES, PER_CU>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES); e != hipSuccess) return e;
    const long nblocks = (long)((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (nblocks > 0x7fffffffL) return hipErrorInvalidValue;
    int blocks = (int)nblocks;
    kern<<<dim3(blocks), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, stream>>>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, nullptr, nullptr, 1);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------------------
// Split-K on 64x64 tiles (and, further down, on 128x128 tiles), for 17 .. 256 rows against a second operand that is too narrow to give every CU a tile: the
// ranges of K of a tile run on different workgroups (see SPLIT_K of hgemm_main_kernel) and meet in a workspace of the
// library's own: one buffer per (device, stream), allocated at first use and replaced by a larger one when a call needs
// more; a buffer that has been handed to a kernel is never freed (a HIP graph captured earlier may hold its address).
// Nothing can be allocated while the stream is capturing: such a call (no buffer yet, or too small a one) takes the
// kernels without split-K instead. The ticket counters, in front of the partial tiles, are zeroed when a buffer is new
// (a fill kernel on the calling stream) and left at zero by every launch.
// ---------------------------------------------------------------------------------------------------------
constexpr size_t kSplitKCounterBytes = 16 * 1024;   // one counter per tile: up to 4096 tiles

static __global__ void hgemm_clear_kernel(unsigned* p, int n) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) p[i] = 0u;
}

static hipError_t split_k_workspace(size_t bytes, hipStream_t stream, char** out, bool* fresh) {
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
    *fresh = false;
    if (b.size < bytes) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &cap);
        if (e != hipSuccess) return e;
        if (cap != hipStreamCaptureStatusNone) return hipErrorStreamCaptureUnsupported;
        const size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes + bytes / 2;
        void* fresh_buf = nullptr;
        e = hipMalloc(&fresh_buf, want);
        if (e != hipSuccess) return e;
        b.ptr = fresh_buf;   // the previous buffer, if any, stays allocated (see above)
        b.size = want;
        *fresh = true;
    }
    *out = static_cast<char*>(b.ptr);
    return hipSuccess;
}

// Number of ranges K is cut into, or 0 where split-K does not apply: 17 .. 256 rows, K a multiple of 64, few enough
// 64x64 tiles for at least four ranges at about two workgroups per CU (up to 128 tiles; up to 192 with a long K), at
// least eight K tiles per range, ranges of equal length. Measured with weights that come from HBM, layout NT (us, without / with split-K): 64 x 4096 x 14336 55 / 32,
// 17 x 4096 x 14336 35 / 29, 128 x 4096 x 14336 54 / 44, 64 x 4096 x 4096 17.4 / 15.7, 96 x 4096 x 4096 17.3 / 15.5,
// 48 x 6144 x 4096 16.6 / 17.4; two ranges only lose (96 x 6144 x 4096 20 / 24, 192 x 4096 x 4096 21 / 25), and so do up to
// 32 rows with a short K, where the small-M kernels are at their best (32 x 4096 x 4096 11 / 15). 129 .. 192 tiles get
// four ranges where K is long (192 x 4096 x 14336 70 / 58, NN 81 / 59; with K = 4096 22 against 21 without; 256 tiles:
// 69 / 73).
static int split_k_ranges(int M, int N, int K) {
    if (M < 17 || M > 256 || K % 64 != 0) return 0;
    if (M <= 32 && K < 8192) return 0;
    const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64);
    if (tiles > 192 || (tiles > 128 && K < 8192)) return 0;
    const int ktiles = K / 64;
    int s = tiles > 128 ? 4 : (int)(512 / tiles);
    if (s > 16) s = 16;
    while (s >= 4 && (ktiles % s != 0 || ktiles / s < 8)) --s;
    return s >= 4 ? s : 0;
}

// The same on 128x128 tiles (64 KiB of partial tile per workgroup), for 193 .. 1024 rows against a long K (the down
// projection): at most 128 tiles, two to four ranges so that about every CU has a workgroup (640 x 3072 x 12288 NT:
// 96 / 76). Measured, weights from HBM
// (us, best tile shape without / with split-K): NT 256 x 4096 x 14336 70 / 54, 384 rows 99 / 83, 512 rows 100 / 86,
// 320 x 2048 x 16384 68 / 47; NN 256 x 4096 x 8192 47 / 38, 384 rows 61 / 54, 512 x 4096 x 14336 108 / 85. Layout NT with
// K = 8192 loses to its 128x64 tiles (384 x 4096 x 8192: 49 / 52), so it needs a longer K; 640 rows (160 tiles) and every
// product with K = 4096 lose 10-60 %.
static int split_k_ranges_128(int M, int N, int K, bool nt) {
    if (M < 193 || M > 1024 || K < (nt ? 12288 : 8192) || K % 64 != 0) return 0;
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    const int ktiles = K / 64;
    if (tiles > 128) {
        // 129 .. 255 tiles leave CUs idle for a whole walk over K. With s ranges the walk takes rounds(s) / s of that time,
        // rounds(s) = ceil(tiles * s / 256), plus about 0.05 s of it for the partial tiles (measured, us without / with: NT
        // 896 x 3072 x 12288, 168 tiles, three ranges 124 / 102; 768 x 4096 x 14336, 192 tiles, four ranges 136 / 130;
        // 768 x 3072 x 12288, 144 tiles, three ranges 123 / 98; 640 x 4096 x 12288, 160 tiles, three ranges 124 / 102;
        // eight ranges lose: 896 x 4096 x 14336 138 / 176, 513 rows 102 / 117): the best s up to four, if it saves 4 %; a
        // saving below 10 % only with a last row of tiles that is at least three quarters full (700 x 4096 x 12288, 192
        // tiles with 60 rows in the last six of every column: 102 / 107)
        if (tiles >= 256 || K < 12288) return 0;
        int best = 0;
        double best_cost = 0.96;
        for (int s = 2; s <= 4; ++s) {
            if (ktiles % s != 0 || ktiles / s < 16) continue;
            const double cost = (double)((tiles * s + 255) / 256) / s + 0.05 * s;
            if (cost < best_cost) { best_cost = cost; best = s; }
        }
        if (best_cost > 0.9 && M % 128 != 0 && M % 128 < 96) return 0;
        return best;
    }
    int s = (int)(256 / tiles);
    if (s > 4) s = 4;
    while (s >= 2 && (ktiles % s != 0 || ktiles / s < 8)) --s;
    return s >= 2 ? s : 0;
}

// hipErrorStreamCaptureUnsupported / hipErrorOutOfMemory: no workspace to be had, the caller takes another kernel
template <typename T, bool A_KC, bool B_KC, int BT = 64, int STAGES = 4, int PER_CU = 2>
static hipError_t launch_split_k(const T* A, const T* B, T* C, const T* R, int M, int N, int K, long lda, long ldb, long ldc,
                                 long ldr, int splits, hipStream_t stream) {
    using Cfg = MainCfg<A_KC, B_KC, BT, BT, 2, 2, STAGES>;
    auto kern = hgemm_main_kernel<T, A_KC, B_KC, BT, BT, 2, 2, 0, true, STAGES, PER_CU, true>;
    static DynamicLdsOnce lds_once;
    if (hipError_t e = lds_once.ensure(reinterpret_cast<const void*>(kern), Cfg::LDS_BYTES); e != hipSuccess) return e;
    const long tiles = (long)((M + BT - 1) / BT) * ((N + BT - 1) / BT);
    if (tiles * sizeof(unsigned) > kSplitKCounterBytes) return hipErrorOutOfMemory;
    const size_t bytes = kSplitKCounterBytes + (size_t)tiles * splits * Cfg::NTHREADS * Cfg::TM * Cfg::TN * 16;
    char* ws = nullptr;
    bool fresh = false;
    if (hipError_t e = split_k_workspace(bytes, stream, &ws, &fresh); e != hipSuccess) return e;
    if (fresh) {
        hgemm_clear_kernel<<<dim3(4), dim3(256), 0, stream>>>(reinterpret_cast<unsigned*>(ws), (int)(kSplitKCounterBytes / sizeof(unsigned)));
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    }
    kern<<<dim3((unsigned)tiles, (unsigned)splits), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES, stream>>>(
        A, B, C, R, M, N, K, lda, ldb, ldc, ldr, reinterpret_cast<float*>(ws + kSplitKCounterBytes), reinterpret_cast<unsigned*>(ws), splits);
    return hipGetLastError();
}

// 17..64 rows: the small-M kernels stream B once per 16 rows (the L2 catches part of the repeats), the 128x128 tiles
// stream it once but run K / 64 dependent tile steps of ~0.4 us on at most one workgroup per 128 columns. Cost models
// from measurements of both at Llama projection shapes; true = the tiles are expected to be faster.
static double small_m_us(int M, int N, int K, bool nn) {
    return (double)((M + 15) / 16) * (double)N * (double)K * 2.0 / 6.5e6 + (nn ? 2.3 : 4.0);
}
static double few_row_tiles_us(int M, int N, int K, bool nt) {
    long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    double step_us = 0.42;
    if (nt && tiles < 192) {   // layout NT runs 128x64 tiles then
        tiles = (long)((M + 127) / 128) * ((N + 63) / 64);
        step_us = 0.34;
    }
    return (double)(K / 64) * step_us * (double)((tiles + 255) / 256);
}
static bool few_rows_prefer_tiles(int M, int N, int K, bool nt) {
    if (M <= 16) return false;
    return few_row_tiles_us(M, N, K, nt) < small_m_us(M, N, K, false) - 4.0;
}
// Which tile shape is expected to finish a product of more than 64 rows first (1 = 256x256, 2 = 128x128, 3 = 64x128 or
// 128x64, 4 = 64x64 two to a CU, 5 = 128x256, 6 = 256x128, 7 = 32x64). A CU takes in 64 bytes per cycle from the memory system, so
// the time of a K tile is set by the tile's bytes as much as by its matrix instructions (the operands of a 128x128 tile
// need the same 512 cycles to arrive that its matrix instructions take): measured cycles per K tile of 64 of one
// workgroup alone on its CU are 2470 (256x256; matrix pipes 2048), 1340 (128x256 and 256x128 on a ring of three stages;
// pipes 1024), 770 (128x128; pipes 512), 576 (half tile) and 384 (64x64). A workgroup spends another 5000-12000 cycles
// outside its K loop (first tiles in flight, epilogue). The workgroups run in rounds of one per CU (two for the 64x64
// tiles); the last round may be a partial one. The model reproduces the measured times of 1024^3 .. 8192^3,
// 2048 x 4096 x 4096 and 1536 x 1536 x 8192 within ~10 %. The 128x128 figure used below is 840, that of the 128x256
// tiles 1400: on N(0,1) operands, under the board's power limit, the larger tiles do better against the smaller ones
// than on zeros (3072 x 3072 x 4096: 75 us against 87 where zeros give 70 against 71). The 128x256 tiles are for the
// products that fill the chip once with them, where 256x256 tiles leave CUs idle and 128x128 tiles need two rounds
// (2048 x 4096 x 4096: 59 us against 66 on 128x128 tiles and 89 on 256x256; 2048 x 4096 x 14336: 186 against 216); of
// the two orientations the one with fewer rounds, 256x128 if they tie (768 x 28672 x 4096: 163 us against 168,
// 1536 x 4096 x 14336: 157 against 161, 768 x 6144 x 4096: 40.7 against 42.1; 2048 x 4096 x 4096 the same either way).
// The 32x64 tiles (ring of 8 stages of 12 KiB, 335 cycles per K tile) are for 65 .. 128 rows against a narrow second
// operand (generation steps of that many sequences through the O and down projections), where 64x64 tiles are only
// half as many as CUs: 128 x 4096 x 14336 NT 41 -> 33 us, 128 x 4096 x 4096 13.2 -> 11.2, 96 x 4096 x 14336 40 -> 32
// (with 256 rows, or 6144 columns, they would need two rounds and lose: 63 us against 45, 20 against 14).
static int cheapest_tile_shape(int M, int N, int K, bool a_k_contiguous, bool nt) {
    struct Cand { int shape, bm, bn, per_cu; double step, fixed; };
    static const Cand cands[] = {{1, 256, 256, 1, 2470., 12000.}, {2, 128, 128, 1, 840., 7000.}, {3, 64, 128, 1, 576., 6000.},
                                 {4, 64, 64, 2, 384., 5000.}, {5, 128, 256, 1, 1400., 9000.}, {6, 256, 128, 1, 1400., 9000.},
                                 {7, 32, 64, 1, 335., 5000.}};
    const double ktiles = (double)((K + 63) / 64);
    int best = 2;
    double best_t = 0.;
    for (const Cand& c : cands) {
        if (c.shape == 7 && !a_k_contiguous) continue;   // 32-row tiles exist for a K-contiguous A only
        const int bm = (c.shape == 3 && nt) ? c.bn : c.bm, bn = (c.shape == 3 && nt) ? c.bm : c.bn;   // layout NT: 128x64
        const long tiles = (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        const long cap = 256L * c.per_cu, full = tiles / cap, rem = tiles % cap;
        double t = (double)full * (c.per_cu * ktiles * c.step + c.fixed);
        if (rem) t += (double)((rem + 255) / 256) * ktiles * c.step + c.fixed;
        if (c.shape == 6) t -= 1.;   // a tie between the two orientations
        if (best_t == 0. || t < best_t) { best_t = t; best = c.shape; }
    }
    return best;
}

// Up to 64 rows on 64x64 tiles with an 8-deep ring: the second operand is streamed once whatever M is, by N / 64
// workgroups that each sustain ~38 GB/s until HBM saturates (~6.3 TB/s); layout NN pays ~10 % for its 128-byte row
// segments. True when that is expected to beat both alternatives above (measured at Llama projection shapes:
// 16 x 14336 x 4096 NT 19 us against 22, 64 rows NN 22 against 31, 64 x 4096 x 4096 NT 15 against 17; but
// 16 x 4096 x 14336 NT 41 against 19 on the split-K small-M kernel, and 16 x 14336 x 4096 NN 21 against 20).
// Layout NT with up to 16 rows always takes the split-K small-M kernel: with weights that are in no cache (a different
// weight matrix on every launch, as in a decoder stack) it is the faster one at every Llama projection shape
// (8 x 28672 x 4096: 39 us against 46, 8 x 14336 x 4096: 23 against 26, 16 x 14336 x 4096: 24.6 against 25.8).
static bool few_rows_prefer_deep_ring(int M, int N, int K, bool nn, bool nt) {
    if (nt && M <= 16) return false;
    const double bytes = (double)N * (double)K * 2.0;
    const double rate = fmin(6.3e6, (double)((N + 63) / 64) * 38e3);   // bytes per microsecond
    const double deep_us = (bytes / rate + 1.0) * (nn ? 1.1 : 1.0);
    double other_us = small_m_us(M, N, K, nn);
    if (M > 16) other_us = fmin(other_us, few_row_tiles_us(M, N, K, nt) + 4.0);
    return deep_us < other_us;
}

template <typename T, bool A_KC, bool B_KC>
static hipError_t launch_layout(const T* A, const T* B, T* C, const T* R, int M, int N, int K, long lda, long ldb,
                                long ldc, long ldr, int variant, hipStream_t stream) {
    // the copies of the fast kernels move 16 bytes into LDS: the operands' rows must be 16-byte aligned. C and the residual
    // may lie anywhere; the kernels that assume whole tiles also assume aligned rows of C (c_aligned).
    const bool ab_aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
                            (lda % 8 == 0) && (ldb % 8 == 0);
    const bool c_aligned = (reinterpret_cast<uintptr_t>(C) % 16 == 0) && (ldc % 8 == 0) &&
                           (reinterpret_cast<uintptr_t>(R) % 16 == 0) && (ldr % 8 == 0);
    const bool aligned = ab_aligned && c_aligned;
    // K that is not a multiple of the tiles' depth (the reference's own tiled kernels take K % 16 == 0,
    // kernels/gemm/pkg/gemm_unified/csrc/auto/gemm_7.cu:115-135): the tiled kernels take any multiple of 8, their
    // prologue handles the K % 64 columns at the end. Up to 64 rows are better served by the small-M kernels, which
    // need whole k-steps: there the last K % 64 columns go through the bounds-checked kernel first, into C, and the
    // product over the first K - K % 64 is added to it as a residual (two roundings more than a single pass; 16 x 4096 x
    // 4104 NT: 10 us, against 16 on tiles). A call that brings a residual of its own takes the tiles.
    if (aligned && R == nullptr && M <= 64 && K > 64 && K % 64 != 0 && variant == 0) {
        const int k_tail = K % 64, k_main = K - k_tail;
        const T* a_tail = A_KC ? A + k_main : A + (long)k_main * lda;
        const T* b_tail = B_KC ? B + k_main : B + (long)k_main * ldb;
        dim3 grid((N + 63) / 64, (M + 63) / 64);
        hgemm_edge_kernel<T, A_KC, B_KC><<<grid, dim3(256), 0, stream>>>(a_tail, b_tail, C, nullptr, M, N, k_tail, lda, ldb, ldc, 0);
        if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
        return launch_layout<T, A_KC, B_KC>(A, B, C, C, M, N, k_main, lda, ldb, ldc, ldc, variant, stream);
    }
    // the tiled kernels address a tile with 32-bit byte offsets: up to 256 rows of lda (ldb) elements
    // Any N: an operand stored [K,N] is copied in 16-byte chunks of its rows, and the chunk that straddles N ends in the
    // padding a leading dimension of a multiple of 8 leaves (what it holds only reaches columns that are never stored).
    const bool ragged_ok = ab_aligned && K % 8 == 0 && K >= 8 && lda < (1L << 22) && ldb < (1L << 22);
    const bool small_m = M <= 64 && !(ragged_ok && few_rows_prefer_tiles(M, N, K, A_KC && B_KC));
    // 17 .. 256 rows against a narrow second operand: split-K, where a workspace is to be had
    if (ragged_ok && variant == 0) {
        if (const int splits = split_k_ranges(M, N, K); splits > 0) {
            const hipError_t e = launch_split_k<T, A_KC, B_KC>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, splits, stream);
            if (e != hipErrorStreamCaptureUnsupported && e != hipErrorOutOfMemory) return e;
            (void)hipGetLastError();
        } else if (const int splits128 = split_k_ranges_128(M, N, K, A_KC && B_KC); splits128 > 0) {
            const hipError_t e = launch_split_k<T, A_KC, B_KC, 128, 0, 1>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, splits128, stream);
            if (e != hipErrorStreamCaptureUnsupported && e != hipErrorOutOfMemory) return e;
            (void)hipGetLastError();
        }
    }
    // 33 .. 64 rows against a second operand of up to 8192 columns (generation steps of that many sequences through the
    // QKV, O and down projections): 32x64 tiles, two rows of up to 128 workgroups. The 64x64 tiles below put half as many
    // workgroups on the stream of the second operand, the small-M kernels stream it once per 16 rows; with weights that
    // come from HBM (us, 64x64 tiles with the 8-deep ring / 32x64 tiles): NT 64 x 4096 x 14336 71 / 55, 48 x 4096 x 4096
    // 19.9 / 15.8, 40 x 6144 x 4096 19.8 / 15.6; NN 64 x 4096 x 14336 84 / 69, 33 x 4096 x 4096 23.5 / 19.5. Up to 32 rows
    // are one row of such tiles, and the small-M kernels stay ahead (NT 32 x 4096 x 14336 37 / 56).
    if constexpr (A_KC) {
        if (ragged_ok && variant == 0 && M > 32 && M <= 64 && (N + 63) / 64 <= 128)
            return launch_main<T, A_KC, B_KC, 32, 64, 2, 2, 0, true, 8>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
    }
    // Up to 64 rows (generation-step projections): 64x64 tiles with an 8-deep ring stream the second operand once, on
    // N / 64 workgroups with ~50 KiB each in flight, where the split-K small-M kernels below stream it once per 16 rows.
    if (ragged_ok && M <= 64 && variant == 0 && few_rows_prefer_deep_ring(M, N, K, A_KC && !B_KC, A_KC && B_KC)) {
        if (M == 64 && N % 64 == 0 && c_aligned) return launch_main<T, A_KC, B_KC, 64, 64, 2, 2>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
        return launch_main<T, A_KC, B_KC, 64, 64, 2, 2, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
    }
    if constexpr (!B_KC) {   // NN and TN
        if (aligned && small_m && K % 32 == 0 && K >= 32 && N % 8 == 0 && ldc % 2 == 0)
            return launch_smallm_nn<T, A_KC>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
    }
    if constexpr (A_KC && B_KC) {
        // (this kernel stores element by element: C and the residual may lie anywhere)
        if (ab_aligned && small_m && K % 64 == 0 && K >= 64) return launch_smallm_nt<T>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
    }
    // Tiled kernels: M and N need not be multiples of the tile, nor of 8. Shapes: 1 = 256x256 (8 waves, ring of 2),
    // 2 = 128x128 (4 waves, ring of 3), 3 = half of that (64x128, for layout NT 128x64, which keeps the 128-byte rows of
    // both K-contiguous operands; ring of 5), 4 = 64x64 with a ring of 4 (64 KiB: two workgroups fit on a CU), 5 = 128x256
    // and 6 = 256x128 (8 waves of 64x64, ring of 3), 7 = 32x64 (4 waves of 16x32, ring of 8; layouts with a K-contiguous
    // A). More than 64 rows: the shape with the least
    // estimated time. Up to 64 rows (products that few_rows_prefer_tiles sends here): 64x64 tiles, two to a CU, for layout
    // NT (17 .. 64 x 28672 x 4096 with weights from HBM: 45 - 52 us against 53 - 57 on 128x64 tiles and 51 on 128x128),
    // 128x128 otherwise (layout NN: 42 - 47 us against 52 - 64).
    if (ragged_ok) {
        int shape = variant >= 1 && variant <= (A_KC ? 7 : 6) ? variant : M <= 64 ? ((A_KC && B_KC) ? 4 : 2) : cheapest_tile_shape(M, N, K, A_KC, A_KC && B_KC);
        const auto whole = [&](int bm, int bn) { return c_aligned && M % bm == 0 && N % bn == 0; };
        switch (shape) {
            case 1:
                if (whole(256, 256)) return launch_main<T, A_KC, B_KC, 256, 256, 2, 4>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                return launch_main<T, A_KC, B_KC, 256, 256, 2, 4, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
            case 3:
                if constexpr (A_KC && B_KC) {
                    if (whole(128, 64)) return launch_main<T, A_KC, B_KC, 128, 64, 2, 2>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                    return launch_main<T, A_KC, B_KC, 128, 64, 2, 2, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                } else {
                    if (whole(64, 128)) return launch_main<T, A_KC, B_KC, 64, 128, 1, 4>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                    return launch_main<T, A_KC, B_KC, 64, 128, 1, 4, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                }
            case 5:
                if (whole(128, 256)) return launch_main<T, A_KC, B_KC, 128, 256, 2, 4>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                return launch_main<T, A_KC, B_KC, 128, 256, 2, 4, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
            case 6:
                if (whole(256, 128)) return launch_main<T, A_KC, B_KC, 256, 128, 4, 2>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                return launch_main<T, A_KC, B_KC, 256, 128, 4, 2, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
            case 7:
                if constexpr (A_KC) return launch_main<T, A_KC, B_KC, 32, 64, 2, 2, 0, true, 8>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                [[fallthrough]];
            case 4:
                if (whole(64, 64)) return launch_main<T, A_KC, B_KC, 64, 64, 2, 2, 0, false, 4, 2>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                return launch_main<T, A_KC, B_KC, 64, 64, 2, 2, 0, true, 4, 2>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
            default:
                if (whole(128, 128)) return launch_main<T, A_KC, B_KC, 128, 128, 2, 2>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
                return launch_main<T, A_KC, B_KC, 128, 128, 2, 2, 0, true>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, stream);
        }
    }
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    hgemm_edge_kernel<T, A_KC, B_KC><<<grid, dim3(256), 0, stream>>>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr);
    return hipGetLastError();
}

// Product with the gate/up epilogue (EPI = 1): N counts the columns of op(B) (twice those of C). Operands that are not
// 16-byte aligned, K that is not a multiple of 64 or N that is not a multiple of 64 report hipErrorNotSupported and the
// caller runs the product and mi355_silu_mul separately.
template <typename T, bool A_KC, bool B_KC>
static hipError_t launch_silu_mul(const T* A, const T* B, T* C, int M, int N, int K, long lda, long ldb,
                                  long ldc, hipStream_t stream) {
    const bool aligned = (reinterpret_cast<uintptr_t>(A) % 16 == 0) && (reinterpret_cast<uintptr_t>(B) % 16 == 0) &&
                         (reinterpret_cast<uintptr_t>(C) % 16 == 0) && (lda % 8 == 0) && (ldb % 8 == 0) && (ldc % 8 == 0);
    // N = columns of op(B); gate/up pairs are 64 columns wide. Few rows are better served by the small-M product.
    if (!aligned || K % 64 != 0 || K < 64 || N % 64 != 0 || lda >= (1L << 22) || ldb >= (1L << 22)) return hipErrorNotSupported;
    if constexpr (A_KC && B_KC) {   // generation step: the split-K small-M kernel with the same epilogue
        if (M <= 16) return launch_smallm_nt_gate_up<T>(A, B, C, M, N, K, lda, ldb, ldc, stream);
    }
    // up to 64 rows (generation steps of a few dozen sequences): 64x64 tiles with an 8-deep ring as for the plain product,
    // four waves side by side along M so that every wave holds the gate and the up columns of its rows
    if (M <= 64 && !few_rows_prefer_tiles(M, N, K, false))
        return launch_main<T, A_KC, B_KC, 64, 64, 4, 1, 1, true>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, stream);
    const bool fits128 = M % 128 == 0 && N % 128 == 0;
    const bool fits256 = M % 256 == 0 && N % 256 == 0;
    const long t256 = (long)((M + 255) / 256) * ((N + 255) / 256);
    if (t256 >= 192) {
        if (fits256) return launch_main<T, A_KC, B_KC, 256, 256, 2, 4, 1>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, stream);
        return launch_main<T, A_KC, B_KC, 256, 256, 2, 4, 1, true>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, stream);
    }
    if (fits128) return launch_main<T, A_KC, B_KC, 128, 128, 2, 2, 1>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, stream);
    return launch_main<T, A_KC, B_KC, 128, 128, 2, 2, 1, true>(A, B, C, nullptr, M, N, K, lda, ldb, ldc, 0, stream);
}

template <typename T>
static hipError_t silu_mul_dispatch_t(const void* A, const void* B, void* C, int M, int N2, int K, long lda, long ldb, long ldc,
                                      int layout, hipStream_t stream) {
    const T* a = static_cast<const T*>(A);
    const T* b = static_cast<const T*>(B);
    T* c = static_cast<T*>(C);
    switch (layout) {
        case MI355_GEMM_NN: return launch_silu_mul<T, true, false>(a, b, c, M, N2, K, lda, ldb, ldc, stream);
        case MI355_GEMM_NT: return launch_silu_mul<T, true, true>(a, b, c, M, N2, K, lda, ldb, ldc, stream);
        default: return hipErrorNotSupported;
    }
}

// MI355_HGEMM_PART: undefined = everything in this translation unit; 0 = the fp16 kernels and the two entry points, 1 =
// only the bf16 kernels behind the two *_bf16 functions (the build compiles the two parts side by side).
hipError_t hgemm_dispatch_bf16(const void* A, const void* B, void* C, const void* R, int M, int N, int K, long lda, long ldb,
                               long ldc, long ldr, int layout, int variant, hipStream_t stream);
hipError_t hgemm_silu_mul_dispatch_bf16(const void* A, const void* B, void* C, int M, int N2, int K, long lda, long ldb,
                                        long ldc, int layout, hipStream_t stream);

#if !defined(MI355_HGEMM_PART) || MI355_HGEMM_PART == 1
hipError_t hgemm_silu_mul_dispatch_bf16(const void* A, const void* B, void* C, int M, int N2, int K, long lda, long ldb,
                                        long ldc, int layout, hipStream_t stream) {
    return silu_mul_dispatch_t<bf16_t>(A, B, C, M, N2, K, lda, ldb, ldc, layout, stream);
}
#endif
#if !defined(MI355_HGEMM_PART) || MI355_HGEMM_PART == 0
hipError_t hgemm_silu_mul_dispatch(const void* A, const void* B, void* C, int M, int N2, int K, long lda, long ldb, long ldc,
                                   int layout, int dtype, hipStream_t stream) {
    if (dtype == MI355_DTYPE_BF16) return hgemm_silu_mul_dispatch_bf16(A, B, C, M, N2, K, lda, ldb, ldc, layout, stream);
    return silu_mul_dispatch_t<half_t>(A, B, C, M, N2, K, lda, ldb, ldc, layout, stream);
}
#endif

template <typename T>
static hipError_t gemm_dispatch_t(const void* A, const void* B, void* C, const void* R, int M, int N, int K, long lda,
                                  long ldb, long ldc, long ldr, int layout, int variant, hipStream_t stream) {
    const T* a = static_cast<const T*>(A);
    const T* b = static_cast<const T*>(B);
    T* c = static_cast<T*>(C);
    const T* r = static_cast<const T*>(R);
    switch (layout) {
        case MI355_GEMM_NN: return launch_layout<T, true, false>(a, b, c, r, M, N, K, lda, ldb, ldc, ldr, variant, stream);
        case MI355_GEMM_NT: return launch_layout<T, true, true>(a, b, c, r, M, N, K, lda, ldb, ldc, ldr, variant, stream);
        case MI355_GEMM_TN: return launch_layout<T, false, false>(a, b, c, r, M, N, K, lda, ldb, ldc, ldr, variant, stream);
        default: return hipErrorInvalidValue;
    }
}

#if !defined(MI355_HGEMM_PART) || MI355_HGEMM_PART == 1
hipError_t hgemm_dispatch_bf16(const void* A, const void* B, void* C, const void* R, int M, int N, int K, long lda, long ldb,
                               long ldc, long ldr, int layout, int variant, hipStream_t stream) {
    return gemm_dispatch_t<bf16_t>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, layout, variant, stream);
}
#endif
#if !defined(MI355_HGEMM_PART) || MI355_HGEMM_PART == 0
hipError_t hgemm_dispatch(const void* A, const void* B, void* C, const void* R, int M, int N, int K, long lda, long ldb,
                          long ldc, long ldr, int layout, int dtype, int variant, hipStream_t stream) {
    if (dtype == MI355_DTYPE_BF16) return hgemm_dispatch_bf16(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, layout, variant, stream);
    return gemm_dispatch_t<half_t>(A, B, C, R, M, N, K, lda, ldb, ldc, ldr, layout, variant, stream);
}
#endif

}  // namespace mi355

#if defined(MI355_TIMELINE) && (!defined(MI355_HGEMM_PART) || MI355_HGEMM_PART == 0)
// profiling build: copies the records of the last tiled fp16 GEMM launch (kMaxWorkgroups x kSlots 64-bit values) to the host
extern "C" int mi355_timeline_read_hgemm(void* dst, size_t bytes) {
    const size_t all = sizeof(unsigned long long) * mi355::timeline::kMaxWorkgroups * mi355::timeline::kSlots;
    return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(mi355::hgemm_stamps), bytes < all ? bytes : all);
}
#endif
