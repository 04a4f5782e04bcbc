// C[M, N] = X[M, K] W[N, K]^T for many rows (prompt portions): bfloat16 operands, float32 accumulation on the
// matrix cores, one rounding at the end (the reference calls cuBLAS here:
// src/ops/kernels/cuda/matmul_kernel.cu:132-154; SwiGLU: src/ops/kernels/cuda/silu_kernel.cu:82-97).
//
// A workgroup of four wavefronts owns an output tile of 256 weight rows x 256 rows of X; every wavefront a quarter
// of it, 128 x 128, as 4 x 4 results of v_mfma_f32_32x32x16_bf16 (256 accumulation registers a lane).  K goes in
// steps of 64 through two LDS stages of 64 KB (the tile's rows of W, then of X, 128 bytes a row) that are filled
// straight from memory (global_load_lds_dwordx4: 16 bytes a lane, a wavefront's 64 pieces to 1 KB of LDS in a row).
//
// The tile of the matrix instruction is taken as D[n][m] = W . X^T: a lane then holds four neighbouring n of one
// row m of C, and, where gate and up rows alternate in slabs of 16, a gate value and its up value in one lane.
//
// What the loop's shape is for (measured on 2,048 x 24,576 x 4,096, all times with the chip warm):
//  * the copies are asked for one at a time between pairs of products, and the operand reads of the next k group
//    likewise: issued in a burst at the head of a step they hold the wavefronts up in the issue queue while the
//    matrix cores idle (a wavefront a SIMD: 335 -> 302 us for the loop alone);
//  * the copies of a step go out over the two quarters behind the barrier that frees their stage, a step and three
//    quarters before they are read (302 -> 292 us);
//  * neither LDS bandwidth (half the operand reads left out: no change) nor the latency of lines that miss L2 (all
//    workgroups on one tile: no change; touching the lines two steps ahead: no change) bounds the loop; the copies'
//    path does (one step in four copied: 271 us), and beyond that the matrix cores at the clock the power limit
//    leaves (no copies and half the reads: 266 us, which is the vendor library's time for the whole product).
// Results leave through LDS, so that rows of the tile are written in whole 16-byte pieces; SwiGLU and the conversion
// happen on the way.  With shares of K (grid-wide, each share a float32 result of its own that the caller's norm
// adds up) a product with few output tiles fills the chip.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

namespace {

constexpr int TILE = 256;                        // weight rows and rows of X a workgroup
constexpr int BK = 64;                           // k a stage
constexpr int ROW_BYTES = BK * 2;                // a row of a stage: eight 16-byte pieces
constexpr int OPERAND_BYTES = TILE * ROW_BYTES;  // 32 KB
constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;   // the tile's rows of W, then of X
constexpr int WAVES_N = 2, WAVES_M = 2;          // wavefronts along the weight rows and along the rows of X
constexpr int NW = WAVES_N * WAVES_M;
constexpr int TN = TILE / 32 / WAVES_N;          // 32-row pieces of W a wavefront
constexpr int TM = TILE / 32 / WAVES_M;          // 32-row pieces of X a wavefront
constexpr int PER = (TILE / 8) / NW;             // 1 KB chunks (8 rows) of an operand's tile a wavefront copies
constexpr int PAIRS = TN * TM / 2;               // pairs of products a k group
constexpr int NR = TN + TM;                      // operand reads a k group
constexpr int PANEL = 8;                         // tiles of X a panel of the tile order

enum { OUT_BF16 = 0, OUT_SWIGLU = 1, OUT_F32 = 2 };

struct TileArgs {
    const bf16_t* X;
    int64_t ldx;
    const bf16_t* W;
    int64_t ldw;
    void* C;
    int64_t ldc;
    int M, N, K;          // K: of one share
    int tiles_m, tiles_n;
    int splits;           // shares of K, each with a result of its own
    int64_t part_stride;  // elements between the shares' results
};

// Piece c of row r of a stage sits at place c ^ swz(r) of the row: the rows that neighbouring lanes read together
// (eight in a row, or sixteen) then lie in different 16-byte places of what LDS serves at once.
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// 16 bytes a lane from memory straight into LDS: lane i's piece, `offset` bytes behind `base`, lands at lds_base + 16 i
// (a wavefront-wide address).  The compiler knows nothing of these copies, so the waits for them are written out below.
__device__ __forceinline__ void load_to_lds(const void* base, uint32_t offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_base), "v"(offset), "s"(base) : "memory", "m0");
}

template <int MODE>
__global__ __launch_bounds__(NW* PULSE_WAVE) void gemm_tile_kernel(TileArgs a) {
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE_BYTES];

    // The workgroups of one die (every eighth workgroup number) take neighbouring tiles, in panels of eight tiles
    // of X, which share their operands in that die's L2; a share of K is a whole set of tiles.
    const int tiles = a.tiles_m * a.tiles_n;
    const int total = tiles * a.splits;
    const int per_die = (total + 7) / 8;
    const int t_all = (blockIdx.x % 8) * per_die + blockIdx.x / 8;
    if (t_all >= total) return;
    const int split = t_all / tiles;
    const int t = t_all - split * tiles;
    const int panel = t / (PANEL * a.tiles_n);
    const int panel_m = min(PANEL, a.tiles_m - panel * PANEL);
    const int in_panel = t - panel * PANEL * a.tiles_n;
    const int tm = panel * PANEL + in_panel % panel_m;
    const int tn = in_panel / panel_m;
    const int m0 = tm * TILE, n0 = tn * TILE;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / PULSE_WAVE);
    const int lane = tid % PULSE_WAVE;
    const int wave_n = wave % WAVES_N, wave_m = wave / WAVES_N;
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (void __attribute__((address_space(3)))*)(&lds[0])));  // the array's address inside LDS

    // Copy: chunk q of a tile is its rows 8 q .. 8 q + 7; lane i brings the piece that belongs at place i % 8 of row
    // i / 8.  Rows past the operand's end are its last row again (their results are not written).
    // The address is a base in scalar registers, which moves along K, and a lane's byte offset from it, which does not.
    const bf16_t* w_base = a.W + static_cast<int64_t>(n0) * a.ldw + static_cast<int64_t>(split) * a.K;
    const bf16_t* x_base = a.X + static_cast<int64_t>(m0) * a.ldx + static_cast<int64_t>(split) * a.K;
    uint32_t w_from[PER], x_from[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int row = (wave * PER + j) * 8 + lane / 8;
        const int c = (lane % 8) ^ swz(row);
        w_from[j] = static_cast<uint32_t>((static_cast<int64_t>(min(n0 + row, a.N - 1) - n0) * a.ldw + c * 8) * 2);
        x_from[j] = static_cast<uint32_t>((static_cast<int64_t>(min(m0 + row, a.M - 1) - m0) * a.ldx + c * 8) * 2);
    }
    auto load_one = [&](int k, int stage, int j) {   // j: first the wavefront's chunks of W, then of X
        const uint32_t to = lds0 + stage * STAGE_BYTES + wave * PER * 1024;
        if (j < PER) load_to_lds(w_base + k, w_from[j], to + j * 1024);
        else load_to_lds(x_base + k, x_from[j - PER], to + OPERAND_BYTES + (j - PER) * 1024);
    };

    // Operand reads: lane l holds row l % 32 and the k group l / 32 (8 values) of a 32 x 16 piece.
    const int h = lane / 32;
    const int e = h ^ swz(lane % 32);
    int w_at[4], x_at[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        const int place = (e ^ (kk << 1)) * 16;
        w_at[kk] = (wave_n * TN * 32 + lane % 32) * ROW_BYTES + place;
        x_at[kk] = OPERAND_BYTES + (wave_m * TM * 32 + lane % 32) * ROW_BYTES + place;
    }
    bf16x8 wf[2][TN], xf[2][TM];
    auto read_one = [&](int stage, int kk, int buf, int r) {
        // (in the order in which the products want them: the pieces of X first, all of which the first pairs take)
        const char* base = lds + stage * STAGE_BYTES;
        if (r < TM) xf[buf][r] = *reinterpret_cast<const bf16x8*>(base + x_at[kk] + r * 32 * ROW_BYTES);
        else wf[buf][r - TM] = *reinterpret_cast<const bf16x8*>(base + w_at[kk] + (r - TM) * 32 * ROW_BYTES);
    };

    f32x16 acc[TN][TM];
#pragma unroll
    for (int f = 0; f < TN; ++f)
#pragma unroll
        for (int g = 0; g < TM; ++g)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[f][g][i] = 0.f;

    // A quarter of a step: the products of one k group from one set of operand registers, in pairs; between the two
    // of a pair one copy instruction (where the quarter has copies), behind the pair its share of the next k group's
    // operand reads into the other set.  Nothing moves across the fences.
    static_assert(PER <= PAIRS, "a copy instruction a pair of products");
    auto quarter = [&](int use, int rd_stage, int rd_kk, int ld_k, int ld_stage, int ld_first) {
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            auto product = [&](int i) {
                acc[i / TM][i % TM] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[use][i / TM], xf[use][i % TM],
                                                                              acc[i / TM][i % TM], 0, 0, 0);
            };
            product(2 * p);
            __builtin_amdgcn_sched_barrier(0);
            if (ld_first >= 0 && p < PER) {
                load_one(ld_k, ld_stage, ld_first + p);
                __builtin_amdgcn_sched_barrier(0);
            }
            product(2 * p + 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = (p * NR + PAIRS - 1) / PAIRS; r < ((p + 1) * NR + PAIRS - 1) / PAIRS; ++r)
                read_one(rd_stage, rd_kk, use ^ 1, r);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // A stage is free once the barrier behind its last reads has passed: the first half of the next copies into it
    // goes out in the quarter right behind that barrier, the second half in the quarter after, and all of them are
    // waited for before the barrier a step later.  Past the end of K the last columns are copied again, for nobody.
    const int steps = a.K / BK;
#pragma unroll
    for (int j = 0; j < 2 * PER; ++j) load_one(0, 0, j);
#pragma unroll
    for (int j = 0; j < PER; ++j) load_one(min(1, steps - 1) * BK, 1, j);
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NR; ++r) read_one(0, 0, 0, r);
    for (int s = 0; s < steps; ++s) {
        const int stage = s & 1;
        quarter(0, stage, 1, min(s + 1, steps - 1) * BK, stage ^ 1, PER);
        quarter(1, stage, 2, 0, 0, -1);
        quarter(0, stage, 3, 0, 0, -1);
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        __syncthreads();
        quarter(1, stage ^ 1, 0, min(s + 2, steps - 1) * BK, stage, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");  // the last copies, which nobody reads, must not land in what follows
    __syncthreads();

    // D[n][m]: lane l holds column m = l % 32 and rows n = 8 (i / 4) + 4 (l / 32) + i % 4, i = 0 .. 15.  Every
    // wavefront turns its results round in a piece of LDS of its own, 32 rows of C at a time, so that whole rows of
    // its part of the tile leave in 16-byte pieces.
    constexpr int WAVE_LDS = 2 * STAGE_BYTES / NW;
    char* mine = lds + wave * WAVE_LDS;
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    const int n_wave = n0 + wave_n * TN * 32;
#pragma unroll
    for (int g = 0; g < TM; ++g) {
        const int m_base = m0 + (wave_m * TM + g) * 32;
        if constexpr (MODE == OUT_BF16 || MODE == OUT_SWIGLU) {
            constexpr int COLS = MODE == OUT_BF16 ? TN * 32 : TN * 16;
            constexpr int PITCH = COLS * 2 + 16;
            static_assert(32 * PITCH <= WAVE_LDS, "a wavefront's piece of LDS holds 32 rows of its part of the tile");
#pragma unroll
            for (int f = 0; f < TN; ++f) {
                if constexpr (MODE == OUT_BF16) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        bf16x4 v;
#pragma unroll
                        for (int i = 0; i < 4; ++i) v[i] = (__bf16)acc[f][g][q * 4 + i];
                        *reinterpret_cast<bf16x4*>(mine + (lane % 32) * PITCH + (f * 32 + q * 8 + h * 4) * 2) = v;
                    }
                } else {
                    // weight rows alternate in slabs of 16: the gate rows of 16 outputs, their up rows behind
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        bf16x4 v;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float gate = acc[f][g][q * 4 + i], up = acc[f][g][8 + q * 4 + i];
                            v[i] = (__bf16)(gate * __builtin_amdgcn_rcpf(1.0f + __expf(-gate)) * up);
                        }
                        *reinterpret_cast<bf16x4*>(mine + (lane % 32) * PITCH + (f * 16 + q * 8 + h * 4) * 2) = v;
                    }
                }
            }
            wave_sync();
            constexpr int PCS = COLS * 2 / 16;       // 16-byte pieces a row
            constexpr int ROWS = PULSE_WAVE / PCS;   // rows an instruction
            bf16_t* out = static_cast<bf16_t*>(a.C);
            const int n_first = MODE == OUT_BF16 ? n_wave : n_wave / 2;
            const int n_end = MODE == OUT_BF16 ? a.N : a.N / 2;
#pragma unroll
            for (int it = 0; it < 32 / ROWS; ++it) {
                const int row = it * ROWS + lane / PCS, pc = lane % PCS;
                const uint4 v = *reinterpret_cast<const uint4*>(mine + row * PITCH + pc * 16);
                const int m = m_base + row, n = n_first + pc * 8;
                if (m < a.M && n < n_end) *reinterpret_cast<uint4*>(out + static_cast<int64_t>(m) * a.ldc + n) = v;
            }
            wave_sync();
        } else {
            constexpr int FP = 2;                    // 32-row pieces of W a pass: 64 float32 columns
            constexpr int PITCH = FP * 32 * 4 + 16;
            static_assert(32 * PITCH <= WAVE_LDS, "a wavefront's piece of LDS holds 32 rows of a pass");
            static_assert(TN % FP == 0, "whole passes");
            float* out = static_cast<float*>(a.C) + split * a.part_stride;
#pragma unroll
            for (int f0 = 0; f0 < TN; f0 += FP) {
#pragma unroll
                for (int f = 0; f < FP; ++f)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float4 v = {acc[f0 + f][g][q * 4], acc[f0 + f][g][q * 4 + 1], acc[f0 + f][g][q * 4 + 2],
                                          acc[f0 + f][g][q * 4 + 3]};
                        *reinterpret_cast<float4*>(mine + (lane % 32) * PITCH + (f * 32 + q * 8 + h * 4) * 4) = v;
                    }
                wave_sync();
                constexpr int PCS = FP * 32 * 4 / 16;
                constexpr int ROWS = PULSE_WAVE / PCS;
#pragma unroll
                for (int it = 0; it < 32 / ROWS; ++it) {
                    const int row = it * ROWS + lane / PCS, pc = lane % PCS;
                    const float4 v = *reinterpret_cast<const float4*>(mine + row * PITCH + pc * 16);
                    const int m = m_base + row, n = n_wave + f0 * 32 + pc * 4;
                    if (m < a.M && n < a.N) *reinterpret_cast<float4*>(out + static_cast<int64_t>(m) * a.ldc + n) = v;
                }
                wave_sync();
            }
        }
    }
}

bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

}  // namespace

// Whether the many-rows product takes these sizes: an inner dimension whose shares are multiples of 64, weight rows
// in multiples of 8 (of 32 with SwiGLU inside, of 4 for float32 results), shares only with float32 results.
extern "C" int pulse_gemm_tile_takes(int M, int N, int K, int mode, int splits) {
    if (M <= 0 || N <= 0 || K <= 0 || splits < 1 || mode < OUT_BF16 || mode > OUT_F32) return 0;
    if (splits > 1 && mode != OUT_F32) return 0;
    if (K % (BK * splits)) return 0;
    const int n_step = mode == OUT_SWIGLU ? 32 : (mode == OUT_BF16 ? 8 : 4);
    if (N % n_step) return 0;
    const int64_t tiles = static_cast<int64_t>((M + TILE - 1) / TILE) * ((N + TILE - 1) / TILE) * splits;
    return tiles <= (1 << 24);
}

// mode 0: C [M, N] bfloat16.  mode 1: the rows of W alternate in slabs of 16 gate rows and their 16 up rows;
// C [M, N / 2] bfloat16 = silu(gate) * up.  mode 2: float32, one result [M, N] for every share of K, `part_stride`
// elements apart (the shares are added up by whoever reads them, in order).
extern "C" int pulse_gemm_tile(const void* X, int64_t ldx, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                               int K, int mode, int splits, int64_t part_stride, void* stream) {
    PULSE_REQUIRE(pulse_gemm_tile_takes(M, N, K, mode, splits),
                  "gemm_tile: %d rows x %d weight rows x inner dimension %d, mode %d, %d shares: the inner dimension must "
                  "be a multiple of 64 a share, the weight rows a multiple of 8 (32 with SwiGLU, 4 for float32 results), "
                  "shares need float32 results", M, N, K, mode, splits);
    PULSE_REQUIRE(X && W && C && aligned16(X) && aligned16(W) && aligned16(C), "gemm_tile: operands must be aligned to 16 bytes");
    PULSE_REQUIRE(ldx >= K && ldw >= K && ldx % 8 == 0 && ldw % 8 == 0 && ldx < (1 << 22) && ldw < (1 << 22),
                  "gemm_tile: rows of X and W must be K long at least, start at multiples of 16 bytes and lie less than "
                  "4M elements apart (strides %lld, %lld)", (long long)ldx, (long long)ldw);
    const int out_cols = mode == OUT_SWIGLU ? N / 2 : N;
    PULSE_REQUIRE(ldc >= out_cols && ldc % (mode == OUT_F32 ? 4 : 8) == 0, "gemm_tile: rows of the result must be %d long at "
                  "least and start at multiples of 16 bytes (stride %lld)", out_cols, (long long)ldc);
    PULSE_REQUIRE(splits == 1 || (part_stride >= static_cast<int64_t>(M - 1) * ldc + N && part_stride % 4 == 0),
                  "gemm_tile: the shares' results overlap (stride %lld)", (long long)part_stride);
    TileArgs a{static_cast<const bf16_t*>(X), ldx, static_cast<const bf16_t*>(W), ldw, C, ldc, M, N, K / splits,
               (M + TILE - 1) / TILE, (N + TILE - 1) / TILE, splits, splits > 1 ? part_stride : 0};
    const dim3 grid(((a.tiles_m * a.tiles_n * splits + 7) / 8) * 8);
    const dim3 block(NW * PULSE_WAVE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mode == OUT_BF16) hipLaunchKernelGGL((gemm_tile_kernel<OUT_BF16>), grid, block, 0, s, a);
    else if (mode == OUT_SWIGLU) hipLaunchKernelGGL((gemm_tile_kernel<OUT_SWIGLU>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((gemm_tile_kernel<OUT_F32>), grid, block, 0, s, a);
    PULSE_LAUNCH_CHECK("gemm_tile");
    return 0;
}
