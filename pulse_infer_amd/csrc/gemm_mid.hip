// C[M, N] = X[M, K] * W[N, K]^T in bfloat16 on the matrix cores for 17 to 192 rows: the regime of decoding with
// many requests and of short prompt portions, where the product still only has to stream the weight from HBM once,
// but X is too large to be fetched again by every wavefront.
//
// A workgroup of four wavefronts owns 64 weight rows (16 a wavefront) and a share of K (grid.y splits K when the
// weight has too few rows to fill the chip otherwise).  The wavefronts walk K together in chunks of 128 (64 from
// 65 rows on, so that two stages of X fit LDS): the chunk of X goes through LDS once for all four, two stages, one
// barrier a chunk; each wavefront
// streams its 16 weight rows straight into registers, whole 128-byte lines per 16 lanes, and brings them into the
// matrix-core layout with DPP and ds_bpermute as the few-rows kernel does.  The weight slab is the row operand and
// X^T the column operand of v_mfma_f32_16x16x32_bf16, so lane l holds output features 4*(l/16)+i of row l%16.
//
// Epilogues: bfloat16 store; SwiGLU of a slab-interleaved (gate, up) weight; float32 partial sums [split, M, N] that a
// consumer adds up in split order (so the result is the same from run to run).  Accumulation is float32
// (reference: cublasGemmEx with CUBLAS_COMPUTE_32F, src/ops/kernels/cuda/matmul_kernel.cu:132-154).
#include "common.h"

#include <math.h>

#include <type_traits>
#include <utility>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int KC_MIN = 128;    // what a share of K must be a multiple of
constexpr int STAGGER_ROWS = 960;    // consecutive weight rows whose owners start at the same chunk of K ..
constexpr int STAGGER_CHUNKS = 4;    // .. this many chunks after the owners of the rows before

template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
// f(integral_constant<int, 0>), .., f(integral_constant<int, N - 1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

enum MidMode : int { MID_BF16 = 0, MID_PARTS = 1 };

__device__ __forceinline__ bf16x8 zeros8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
}

// NW wavefronts of 16 weight rows each a workgroup; MT tiles of 16 rows of X; KC k a chunk (steps of 32); RING
// register sets of weight chunks (a wavefront has RING - 1 chunks of its 16 weight rows in flight).
template <int NW, int MT, int KC, bool SWIGLU, int RING>
__global__ __launch_bounds__(NW* PULSE_WAVE) void gemm_mid_kernel(const bf16_t* __restrict__ X, int64_t ldx,
                                                                    const bf16_t* __restrict__ W, int64_t ldw,
                                                                    void* __restrict__ C, int64_t ldc, int M, int N,
                                                                    int k_len, int mode) {
    constexpr int XROW = KC + 8;   // bfloat16 a row of X takes in LDS: 16 bytes of padding spread the rows over the banks
    __shared__ __attribute__((aligned(16))) bf16_t s_x[2][16 * MT * XROW];
    static_assert(!SWIGLU || NW % 2 == 0, "gate and up slabs come in pairs");
    static_assert(KC == 64 || KC == 128, "a chunk is one or two pairs of steps");
    static_assert(sizeof(f32x4) * (NW / 2) * MT * PULSE_WAVE <= sizeof(bf16_t) * 2 * 16 * MT * XROW,
                  "the up slabs' results take the place of the stages of X at the end");
    constexpr int NT = 16 * NW;                                  // weight rows of a workgroup
    constexpr int THREADS = NW * PULSE_WAVE;
    constexpr int ROWP = KC / 8;                                 // 16-byte pieces of a row of a chunk of X
    constexpr int PIECES = 16 * MT * ROWP;
    constexpr int XP = (PIECES + THREADS - 1) / THREADS;         // pieces a thread stages
    constexpr int PAIRS = KC / 64;                               // pairs of steps a chunk

    const int tid = threadIdx.x;
    const int wave = tid / PULSE_WAVE;
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;
    const int n_base = blockIdx.x * NT;
    const int split = blockIdx.y;
    const int64_t k0 = static_cast<int64_t>(split) * k_len;
    const int chunks = k_len / KC;
    // Workgroups do not all walk their share of K from the same end: the owners of every 960 weight rows start four
    // chunks later than the owners of the 960 before (and wrap around), which loads the memory channels more evenly
    // (gate+up of the 8B shape: 5 to 9% faster).  The order of the sums depends on the weight row and the share only,
    // not on the workgroup's shape (960 is a multiple of the rows of every shape: 32, 48, 64, 96, 160) or on X.
    const int rot = static_cast<int>(((n_base / STAGGER_ROWS) * STAGGER_CHUNKS + blockIdx.y) % static_cast<unsigned>(chunks));
    auto placed = [&](int c) { return c + rot >= chunks ? c + rot - chunks : c + rot; };  // where chunk c of the walk lies

    // Weight loads: 16 consecutive lanes fetch two whole 128-byte lines (rows 2kg + r/8 and that + 8, piece r%8);
    // rows beyond N repeat the last row: their products only reach outputs that are never stored.
    const int wrow = n_base + 16 * wave + 2 * kg + (r >> 3);
    const bf16_t* w0 = W + static_cast<int64_t>(min(wrow, N - 1)) * ldw + k0 + (r & 7) * 8;
    const bf16_t* w1 = W + static_cast<int64_t>(min(wrow + 8, N - 1)) * ldw + k0 + (r & 7) * 8;
    // after the exchange of halves, lane (q, i) holds row 2q + i/8 + 8 * (i/4 % 2) and k-group i % 4 of a step;
    // the operand's lane (kg, r) takes it from there
    const int source_lane = 16 * ((r >> 1) & 3) + 8 * (r & 1) + 4 * (r >> 3) + kg;

    // X pieces (16 bytes) of a chunk that this thread stages: piece p = tid + THREADS i is row p / ROWP, columns
    // 8 (p % ROWP)..; xdst < 0: no such piece
    // Every load of the walk is issued whatever the thread, the row or the chunk: a load under a condition would keep
    // the compiler from counting the loads in flight, and it would wait for all of them before every chunk (which
    // undoes the ring).  So rows beyond M repeat row M - 1 (their products only reach outputs that are never
    // stored; a thread without a piece to stage fetches from that row too), and chunks beyond the last one fetch
    // the last one again.
    const bf16_t* xsrc[XP];
    int xdst[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int p = tid + THREADS * i;
        const int xr = p / ROWP, xc = p % ROWP;
        xsrc[i] = X + static_cast<int64_t>(min(xr, M - 1)) * ldx + k0 + xc * 8;
        xdst[i] = p < PIECES ? xr * XROW + xc * 8 : -1;
    }

    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Loads run ahead of their use by more than a trip to memory: the weight RING - 1 chunks (a ring of register
    // sets), X two chunks (two sets; X comes from L2 for every workgroup but the first).
    bf16x8 xg[2][XP];
    bf16x8 wr[RING][2 * PAIRS];
    auto load_x = [&](int c, bf16x8 (&x)[XP]) {
        const int64_t at = static_cast<int64_t>(placed(min(c, chunks - 1))) * KC;
#pragma unroll
        for (int i = 0; i < XP; ++i) x[i] = *reinterpret_cast<const bf16x8*>(xsrc[i] + at);
    };
    auto load_w = [&](int c, bf16x8 (&w)[2 * PAIRS]) {
        const int64_t at = static_cast<int64_t>(placed(min(c, chunks - 1))) * KC;
#pragma unroll
        for (int pair = 0; pair < PAIRS; ++pair) {
            w[2 * pair] = __builtin_bit_cast(bf16x8, stream_load16(w0 + at + pair * 64));
            w[2 * pair + 1] = __builtin_bit_cast(bf16x8, stream_load16(w1 + at + pair * 64));
        }
    };
    // One chunk (J = its number modulo RING, which names its register sets): X into its stage, loads for later chunks
    // on their way, then the products of this one.
    auto body = [&](auto J, int c) {
        constexpr int j = decltype(J)::value;
        bf16_t* stage = s_x[c & 1];
#pragma unroll
        for (int i = 0; i < XP; ++i)
            if (xdst[i] >= 0) *reinterpret_cast<bf16x8*>(stage + xdst[i]) = xg[j % 2][i];
        // Everybody has left the chunk before the last one (they passed the barrier of the last one), whose stage
        // this is; after this barrier everybody sees this chunk.
        __syncthreads();
        load_x(c + 2, xg[j % 2]);
        load_w(c + RING - 1, wr[(j + RING - 1) % RING]);
#pragma unroll
        for (int pair = 0; pair < PAIRS; ++pair) {
            const i32x4 l0 = __builtin_bit_cast(i32x4, wr[j][2 * pair]);
            const i32x4 l1 = __builtin_bit_cast(i32x4, wr[j][2 * pair + 1]);
            i32x4 a0, a1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // lanes 4-7 and 12-15 of a row of 16 take the first half-line of rows 8-15 from four lanes below
                const int first = __builtin_amdgcn_update_dpp(l0[e], l1[e], 0x114 /* row_shr:4 */, 0xF, 0xA, false);
                // lanes 0-3 and 8-11 take the second half-line of rows 0-7 from four lanes above
                const int second = __builtin_amdgcn_update_dpp(l1[e], l0[e], 0x104 /* row_shl:4 */, 0xF, 0x5, false);
                a0[e] = __builtin_amdgcn_ds_bpermute(source_lane * 4, first);
                a1[e] = __builtin_amdgcn_ds_bpermute(source_lane * 4, second);
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const bf16x8 a = __builtin_bit_cast(bf16x8, h == 0 ? a0 : a1);
                const int ks = 2 * pair + h;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const bf16x8 xb = *reinterpret_cast<const bf16x8*>(stage + (16 * mt + r) * XROW + ks * 32 + kg * 8);
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, xb, acc[mt], 0, 0, 0);
                }
            }
        }
    };

    load_x(0, xg[0]);
    load_w(0, wr[0]);
    load_x(1, xg[1]);
    static_for<RING - 2>([&](auto J) { load_w(decltype(J)::value + 1, wr[decltype(J)::value + 1]); });
    int c = 0;
    for (; c + RING <= chunks; c += RING)   // whole turns of the ring without a branch inside
        static_for<RING>([&](auto J) { body(J, c + decltype(J)::value); });
    static_for<RING - 1>([&](auto J) {
        if (c + decltype(J)::value < chunks) body(J, c + decltype(J)::value);
    });

    // lane (kg, r) holds features n_base + 16 wave + 4 kg + i of row 16 mt + r
    if (!SWIGLU) {
        const int n = n_base + 16 * wave + 4 * kg;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = 16 * mt + r;
            if (m >= M || n >= N) continue;
            if (mode == MID_PARTS) {
                float* dst = static_cast<float*>(C) + (static_cast<int64_t>(split) * M + m) * ldc + n;
                if (n + 3 < N) *reinterpret_cast<f32x4*>(dst) = acc[mt];
                else
                    for (int i = 0; i < 4 && n + i < N; ++i) dst[i] = acc[mt][i];
            } else {
                bf16_t* dst = static_cast<bf16_t*>(C) + static_cast<int64_t>(m) * ldc + n;
                if (n + 3 < N) {
                    bf16x4 v;
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = (__bf16)acc[mt][i];
                    *reinterpret_cast<bf16x4*>(dst) = v;
                } else {
                    for (int i = 0; i < 4 && n + i < N; ++i) dst[i] = f32_to_bf16(acc[mt][i]);
                }
            }
        }
    } else {
        // even wavefronts hold gate slabs, odd ones the up slabs beside them; the output has half as many columns.
        // The up slabs' results go through the memory of the stages of X, which everybody has left after a barrier.
        f32x4 (*s_up)[MT][PULSE_WAVE] = reinterpret_cast<f32x4 (*)[MT][PULSE_WAVE]>(&s_x[0][0]);
        __syncthreads();
        if (wave & 1) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) s_up[wave / 2][mt][lane] = acc[mt];
        }
        __syncthreads();
        if (!(wave & 1)) {
            const int n = n_base / 2 + 16 * (wave / 2) + 4 * kg;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int m = 16 * mt + r;
                if (m >= M || 2 * n >= N) continue;
                const f32x4 up = s_up[wave / 2][mt][lane];
                bf16_t* dst = static_cast<bf16_t*>(C) + static_cast<int64_t>(m) * ldc + n;
                bf16x4 v;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g = acc[mt][i];
                    v[i] = (__bf16)(g / (1.0f + expf(-g)) * up[i]);
                }
                *reinterpret_cast<bf16x4*>(dst) = v;   // N is a multiple of 32: whole groups of four
            }
        }
    }
}

// Weight loads run three chunks of 128 k ahead (512 / KC slots of the ring). Seven chunks ahead for workgroups of two
// wavefronts, which are taken where the weight has few rows, was measured and changed nothing (6,144 weight rows at
// 64 rows of X: 20.8 us with either depth), so every shape keeps the shallow ring and its registers.
template <int NW, int KC>
constexpr int ring_for() { return 512 / KC; }

template <int NW, int MT, int KC = 128>
void launch_mid(const bf16_t* X, int64_t ldx, const bf16_t* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                int k_len, int splits, int mode, bool swiglu, hipStream_t stream) {
    const dim3 grid((N + 16 * NW - 1) / (16 * NW), splits);
    const dim3 block(NW * PULSE_WAVE);
    constexpr int RING = ring_for<NW, KC>();
    if constexpr (NW % 2 == 0) {
        if (swiglu) {
            hipLaunchKernelGGL((gemm_mid_kernel<NW, MT, KC, true, RING>), grid, block, 0, stream, X, ldx, W, ldw, C, ldc, M, N, k_len, mode);
            return;
        }
    }
    hipLaunchKernelGGL((gemm_mid_kernel<NW, MT, KC, false, RING>), grid, block, 0, stream, X, ldx, W, ldw, C, ldc, M, N, k_len, mode);
}

template <int NW>
void launch_rows(const bf16_t* X, int64_t ldx, const bf16_t* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                 int k_len, int splits, int mode, bool swiglu, hipStream_t stream) {
    if (M <= 16) launch_mid<NW, 1>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
    else if (M <= 32) launch_mid<NW, 2>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
    else if (M <= 48) launch_mid<NW, 3>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
    else launch_mid<NW, 4>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
}

// 65 to 192 rows: four or six wavefronts, chunks of 64 k, rows rounded up to 32
template <int NW>
void launch_many_rows(const bf16_t* X, int64_t ldx, const bf16_t* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                      int k_len, int splits, int mode, bool swiglu, hipStream_t stream) {
    if (M <= 96) launch_mid<NW, 6, 64>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
    else if (M <= 128) launch_mid<NW, 8, 64>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
    else if (M <= 160) launch_mid<NW, 10, 64>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
    else launch_mid<NW, 12, 64>(X, ldx, W, ldw, C, ldc, M, N, k_len, splits, mode, swiglu, stream);
}

}  // namespace

// Whether pulse_gemm_mid takes a shape: 1..192 rows, K cut into `splits` shares that are multiples of 128.
extern "C" int pulse_gemm_mid_takes(int M, int N, int K, int splits) {
    return M >= 1 && M <= 192 && N > 0 && K > 0 && splits >= 1 && splits <= 64 && K % splits == 0 && (K / splits) % KC_MIN == 0;
}

// mode 0: C is bfloat16 [M, N] (splits must be 1).  mode 1: C is float32 [splits, M, N] (row stride ldc), the partial
// products of the shares of K, to be added up by the consumer in split order.  swiglu != 0 (mode 0, splits 1): W holds
// gate and up rows interleaved in slabs of 16 (gate slab, up slab, ...), N counts both, C is bfloat16 [M, N / 2] =
// silu(gate) * up.
// waves: wavefronts (of 16 weight rows) a workgroup, 2, 3, 4, 6 or 10 (4 or 6 above 64 rows); 0 lets the entry point choose.
extern "C" int pulse_gemm_mid(const void* X, int64_t ldx, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                              int K, int mode, int swiglu, int splits, int waves, hipStream_t stream) {
    PULSE_REQUIRE(pulse_gemm_mid_takes(M, N, K, splits), "gemm_mid: M=%d (1..192) N=%d K=%d in %d shares (multiples of %d)",
                  M, N, K, splits, KC_MIN);
    PULSE_REQUIRE(X && W && C, "gemm_mid: null pointer");
    PULSE_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K, "gemm_mid: the row strides must be multiples of 8 and cover K");
    PULSE_REQUIRE((reinterpret_cast<uintptr_t>(X) % 16) == 0 && (reinterpret_cast<uintptr_t>(W) % 16) == 0 &&
                  (reinterpret_cast<uintptr_t>(C) % 16) == 0, "gemm_mid: operands must be 16-byte aligned");
    PULSE_REQUIRE(mode == MID_BF16 || mode == MID_PARTS, "gemm_mid: unknown output mode %d", mode);
    PULSE_REQUIRE(mode == MID_PARTS || splits == 1, "gemm_mid: a bfloat16 result needs all of K in one share");
    PULSE_REQUIRE(ldc % 4 == 0, "gemm_mid: the output's row stride must be a multiple of 4");
    if (swiglu) {
        PULSE_REQUIRE(mode == MID_BF16 && N % 32 == 0 && ldc >= N / 2, "gemm_mid: SwiGLU needs N %% 32 == 0 and bfloat16 output");
    } else {
        PULSE_REQUIRE(ldc >= N, "gemm_mid: output row stride too small");
    }
    const bf16_t* x = static_cast<const bf16_t*>(X);
    const bf16_t* w = static_cast<const bf16_t*>(W);
    const int k_len = K / splits;
    if (waves == 0) waves = 4;
    // (16 x waves divides the 960 rows of a stagger group, so the order of a row's sums does not depend on the shape)
    PULSE_REQUIRE(waves == 2 || waves == 3 || waves == 4 || waves == 6 || waves == 10,
                  "gemm_mid: 2, 3, 4, 6 or 10 wavefronts a workgroup, got %d", waves);
    PULSE_REQUIRE(!swiglu || waves % 2 == 0, "gemm_mid: SwiGLU needs an even number of wavefronts");
    PULSE_REQUIRE(M <= 64 || waves == 4 || waves == 6, "gemm_mid: more than 64 rows take 4 or 6 wavefronts a workgroup, got %d", waves);
    if (M > 64 && waves == 6) launch_many_rows<6>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    else if (M > 64) launch_many_rows<4>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    else if (waves == 2) launch_rows<2>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    else if (waves == 3) launch_rows<3>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    else if (waves == 4) launch_rows<4>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    else if (waves == 6) launch_rows<6>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    else launch_rows<10>(x, ldx, w, ldw, C, ldc, M, N, k_len, splits, mode, swiglu != 0, stream);
    PULSE_LAUNCH_CHECK("gemm_mid");
    return 0;
}
