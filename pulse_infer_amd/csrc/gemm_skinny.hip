// C[M, N] = X[M, K] * W[N, K]^T for few rows (M <= 64) in bfloat16 on the matrix
// cores: the regime of decoding, where the product only has to stream the
// weight from HBM once.
//
// A workgroup of KW wavefronts owns SLABS slabs of 16 weight rows.  Each
// wavefront takes its share of K and runs v_mfma_f32_16x16x32_bf16 with the
// weight slab as the row operand and X^T as the column operand (both are 16-byte
// loads of 8 consecutive k), so the result is C^T: lane l holds output features
// 4*(l/16)+i of row l%16.  The wavefronts' partial tiles are summed through LDS in
// wavefront order, so the result is the same from run to run.  The epilogue
// stores bfloat16 or float32, adds into a float32 matrix (the residual), or
// applies SwiGLU to a (gate, up) pair of slabs of a slab-interleaved weight.
// Accumulation is float32 (reference: cublasGemmEx with CUBLAS_COMPUTE_32F,
// src/ops/kernels/cuda/matmul_kernel.cu:132-154).
#include "common.h"

#include <math.h>

namespace {

constexpr int UNROLL = 8;
constexpr int XLDS_BYTES = 16384;  // the most LDS a workgroup takes for X: more costs occupancy and gains nothing

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;

enum OutMode : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_ADD_F32 = 2 };

__device__ __forceinline__ bf16x8 zeros8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
}

// Lane i of a row of 16 lanes takes the value of lane i + N; lanes without a source take zero.
template <int N>
__device__ __forceinline__ int row_shift_left(int v) {
    return __builtin_amdgcn_update_dpp(0, v, 0x100 + N /* row_shl:N */, 0xF, 0xF, true);
}

__device__ __forceinline__ int row_shift_left(int v, int n) {
    switch (n) {  // n is a constant after unrolling: the switch folds to one instruction
        case 1: return row_shift_left<1>(v);
        case 2: return row_shift_left<2>(v);
        case 3: return row_shift_left<3>(v);
        case 4: return row_shift_left<4>(v);
        case 5: return row_shift_left<5>(v);
        case 6: return row_shift_left<6>(v);
        case 7: return row_shift_left<7>(v);
        case 8: return row_shift_left<8>(v);
        case 9: return row_shift_left<9>(v);
        case 10: return row_shift_left<10>(v);
        case 11: return row_shift_left<11>(v);
        case 12: return row_shift_left<12>(v);
        case 13: return row_shift_left<13>(v);
        case 14: return row_shift_left<14>(v);
        case 15: return row_shift_left<15>(v);
        default: return v;
    }
}

// Sum of the wavefronts' partial tiles, in wavefront order, and the store.  With `sumsq` (adding into a float32
// matrix only) every slab also leaves the sum of squares of its 16 new values of each row, sumsq[row * parts + slab
// number]: what a following RMSNorm needs of the row, so that the product after it can normalise by itself; `copy`
// takes the new values once more, each multiplied by its column's `copy_scale` (that norm's weight; null: 1) and
// rounded to bfloat16 (that product's input).  `row_scale` (one factor for each of at most 16 rows) multiplies the
// sums before anything else is done with them.
template <int SLABS, int MT, int KW, bool SWIGLU>
__device__ __forceinline__ void epilogue(float (*red)[SLABS * MT][16][17], void* __restrict__ C, int64_t ldc, int M, int N,
                                         int n_base, int mode, int tid, float* __restrict__ sumsq = nullptr, int parts = 0,
                                         const float* row_scale = nullptr, bf16_t* __restrict__ copy = nullptr,
                                         int64_t ldcopy = 0, const bf16_t* __restrict__ copy_scale = nullptr) {
    constexpr int TILES = SLABS * MT;
    constexpr int THREADS = KW * PULSE_WAVE;
    if (!SWIGLU) {
        for (int e = tid; e < TILES * 256; e += THREADS) {
            const int tile = e / 256;
            const int m_in = (e % 256) / 16;
            const int n_in = e % 16;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < KW; ++w) v += red[w][tile][n_in][m_in];
            if (row_scale) v *= row_scale[m_in];
            const int m = (tile % MT) * 16 + m_in;
            const int n = n_base + (tile / MT) * 16 + n_in;
            float updated = 0.f;
            if (m < M && n < N) {
                const int64_t at = static_cast<int64_t>(m) * ldc + n;
                if (mode == OUT_BF16) static_cast<bf16_t*>(C)[at] = f32_to_bf16(v);
                else if (mode == OUT_F32) static_cast<float*>(C)[at] = v;
                else {
                    updated = static_cast<float*>(C)[at] + v;
                    static_cast<float*>(C)[at] = updated;
                    if (copy)
                        copy[static_cast<int64_t>(m) * ldcopy + n] =
                            f32_to_bf16(copy_scale ? updated * bf16_to_f32(copy_scale[n]) : updated);
                }
            }
            if (sumsq) {  // the 16 lanes of a row of lanes hold the 16 columns of one row of the tile
                float sq = updated * updated;
                sq += __shfl_xor(sq, 8, 16);
                sq += __shfl_xor(sq, 4, 16);
                sq += __shfl_xor(sq, 2, 16);
                sq += __shfl_xor(sq, 1, 16);
                if (n_in == 0 && m < M) sumsq[static_cast<int64_t>(m) * parts + n_base / 16 + tile / MT] = sq;
            }
        }
    } else {
        // slabs come in (gate, up) pairs; the output has half as many columns
        constexpr int PAIRS = SLABS / 2;
        for (int e = tid; e < PAIRS * MT * 256; e += THREADS) {
            const int pt = e / 256;  // pair * MT + mt
            const int m_in = (e % 256) / 16;
            const int n_in = e % 16;
            const int pair = pt / MT, mt = pt % MT;
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int w = 0; w < KW; ++w) {
                g += red[w][(2 * pair) * MT + mt][n_in][m_in];
                u += red[w][(2 * pair + 1) * MT + mt][n_in][m_in];
            }
            if (row_scale) {
                g *= row_scale[m_in];
                u *= row_scale[m_in];
            }
            const int m = mt * 16 + m_in;
            const int n = n_base / 2 + pair * 16 + n_in;
            if (m < M && 2 * n < N) {  // N counts gate and up rows together
                const float v = g / (1.0f + expf(-g)) * u;
                static_cast<bf16_t*>(C)[static_cast<int64_t>(m) * ldc + n] = f32_to_bf16(v);
            }
        }
    }
}

// SLABS slabs of 16 weight rows a workgroup, MT tiles of 16 rows of X, KW wavefronts sharing K.
// XLDS: X (at most 16 rows, MT == 1) is first copied into LDS in operand order, so that the loop's only global
// loads are the weight's.  Without it, lanes whose row of X does not exist skip their load: the cost of the X loads
// is per active lane, and it is what keeps this kernel from the speed of a plain read of the weight.
template <int SLABS, int MT, int KW, bool SWIGLU, bool XLDS>
__global__ __launch_bounds__(KW* PULSE_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ X, int64_t ldx,
                                                                      const bf16_t* __restrict__ W, int64_t ldw,
                                                                      void* __restrict__ C, int64_t ldc, int M, int N,
                                                                      int K, int mode) {
    constexpr int TILES = SLABS * MT;
    constexpr int THREADS = KW * PULSE_WAVE;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // the partial tiles reuse the room of X once every wavefront is done with it
    float (*red)[TILES][16][17] = reinterpret_cast<float (*)[TILES][16][17]>(smem);
    bf16x8* xs = reinterpret_cast<bf16x8*>(smem);  // [K / 8][M]

    const int tid = threadIdx.x;
    const int wave = tid / PULSE_WAVE;
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;
    const int n_base = blockIdx.x * SLABS * 16;

    const int steps = (K + 31) / 32;
    const int per = (steps + KW - 1) / KW;
    const int step_begin = wave * per;
    const int step_end = min(steps, step_begin + per);

    if (XLDS) {
        const int k8s = K / 8;
        for (int c = tid; c < k8s * M; c += THREADS) {
            const int m = c / k8s, k8 = c - m * k8s;
            xs[k8 * M + m] = *reinterpret_cast<const bf16x8*>(X + static_cast<int64_t>(m) * ldx + k8 * 8);
        }
        __syncthreads();
    }

    f32x4 acc[SLABS][MT];
#pragma unroll
    for (int s = 0; s < SLABS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // rows beyond N read row 0: their products only reach outputs that are never stored
    const bf16_t* wrow[SLABS];
#pragma unroll
    for (int s = 0; s < SLABS; ++s) {
        const int n = n_base + s * 16 + r;
        wrow[s] = W + static_cast<int64_t>(n < N ? n : 0) * ldw;
    }
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xok[mt] = m < M;
        xrow[mt] = X + static_cast<int64_t>(xok[mt] ? m : 0) * ldx;
    }
    const int xm = r < M ? r : 0;  // XLDS: the row this lane reads (rows that do not exist repeat row 0)

    // Whole groups of UNROLL k-steps first: all their loads are issued before the first product waits for one,
    // and nothing is done to a loaded value in between (a select on it would make every load wait).
    const int whole_steps = K / 32;  // steps that lie inside K entirely
    int ks = step_begin;
    for (; ks + UNROLL <= min(step_end, whole_steps); ks += UNROLL) {
        bf16x8 xb[UNROLL][MT], wa[UNROLL][SLABS];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k = (ks + u) * 32 + kg * 8;
#pragma unroll
            for (int s = 0; s < SLABS; ++s) wa[u][s] = *reinterpret_cast<const bf16x8*>(wrow[s] + k);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (XLDS) {
                    xb[u][mt] = xs[(k / 8) * M + xm];
                } else {
                    xb[u][mt] = zeros8();
                    if (xok[mt]) xb[u][mt] = *reinterpret_cast<const bf16x8*>(xrow[mt] + k);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int s = 0; s < SLABS; ++s)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u][s], xb[u][mt], acc[s][mt], 0, 0, 0);
    }
    // what is left, one step at a time; the last step may reach beyond K
    for (; ks < step_end; ++ks) {
        const int k = ks * 32 + kg * 8;
        const bool kok = k < K;
        const int kc = kok ? k : 0;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            bf16x8 xb = zeros8();
            if (kok && xok[mt]) xb = XLDS ? xs[(kc / 8) * M + xm] : *reinterpret_cast<const bf16x8*>(xrow[mt] + kc);
#pragma unroll
            for (int s = 0; s < SLABS; ++s) {
                bf16x8 wa = zeros8();
                if (kok) wa = *reinterpret_cast<const bf16x8*>(wrow[s] + kc);
                acc[s][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb, acc[s][mt], 0, 0, 0);
            }
        }
    }

    if (XLDS) __syncthreads();  // every wavefront has read its part of X; its room now takes the partial tiles
#pragma unroll
    for (int s = 0; s < SLABS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][s * MT + mt][4 * kg + i][r] = acc[s][mt][i];
    __syncthreads();

    epilogue<SLABS, MT, KW, SWIGLU>(red, C, ldc, M, N, n_base, mode, tid);
}

// The streaming kernel for at most 16 rows of X when K is a multiple of 256 * KW (every wavefront then runs whole
// groups of UNROLL k-steps).  Two things set it apart from the kernel above:
//
//  * Weight loads are contiguous.  The matrix-core operand wants 16 rows x 16 bytes from every 16 consecutive
//    lanes, which costs a memory request a lane.  Here 16 consecutive lanes fetch two whole 128-byte lines
//    instead: two k-steps (64 values of k) of a slab are two loads of 8 rows x 128 bytes, load h giving lane
//    (q = lane / 16, i = lane % 16) row 2q + i/8 + 8h and the i%8-th 16 bytes of the line.  A DPP move by four
//    lanes then trades the halves of the lines between the two registers (register = k-step afterwards), and one
//    ds_bpermute a register brings every value to the lane whose row and k-group the operand expects.
//  * X loads are packed.  With M <= 16 / PACK rows, the 16 column lanes of the X^T operand hold PACK consecutive
//    k-steps of the same rows (lane c: row c % (16 / PACK), k-step c / (16 / PACK)), so one load serves PACK steps
//    and a DPP shift hands each step its columns.  Columns beyond M read as zero.  (Contiguous loads of X with a
//    ds_bpermute a step were measured too and gain nothing.)
//
// Both only change which lane fetches what; every product and the order of the sums are those of the kernel above.
//
// SCALED: X is a matrix whose rows have not been normalised yet (a bfloat16 copy of the residual, already multiplied
// by the norm's weight, column by column); the sums of squares of the residual's rows that the product before left
// come with it (`sumsq`, `parts` of them a row), and every row of the result is multiplied by 1 / sqrt(mean + eps)
// in the epilogue, where it costs nothing: x W^T scaled by rows is (x scaled by rows) W^T.  That saves the norm
// kernel's launch.  (Forming the normalised x in this kernel's loop from the float32 residual was measured too: every k-step
// then reads float32 values and a weight of the norm, and from 8 rows on that costs what the launch saves.)
constexpr int STAGGER_BLOCKS = 64;  // consecutive workgroups that start at the same group of k-steps

struct RowScale {
    const float* sumsq;  // [M, parts]
    int parts;
    float eps;
};

template <int SLABS, int KW, int PACK, bool SWIGLU, bool SCALED>
__global__ __launch_bounds__(KW* PULSE_WAVE) void gemm_skinny_stream_kernel(const bf16_t* __restrict__ X, int64_t ldx,
                                                                             const bf16_t* __restrict__ W, int64_t ldw,
                                                                             void* __restrict__ C, int64_t ldc, int M,
                                                                             int N, int K, int mode, RowScale scale,
                                                                             float* __restrict__ sumsq_out, int parts_out,
                                                                             bf16_t* __restrict__ copy_out, int64_t ldcopy,
                                                                             const bf16_t* __restrict__ copy_scale) {
    constexpr int THREADS = KW * PULSE_WAVE;
    static_assert(PACK == 1 || PACK == 2 || PACK == 4 || PACK == 8, "PACK k-steps a load of X");
    static_assert(UNROLL % 2 == 0 && UNROLL % PACK == 0, "groups hold whole pairs and whole packs");
    constexpr int MP = 16 / PACK;  // rows of X a pack has room for
    extern __shared__ __attribute__((aligned(16))) char smem[];
    float (*red)[SLABS][16][17] = reinterpret_cast<float (*)[SLABS][16][17]>(smem);

    const int tid = threadIdx.x;
    const int wave = tid / PULSE_WAVE;
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;
    const int n_base = blockIdx.x * SLABS * 16;
    const int per = K / 32 / KW;  // a multiple of UNROLL (checked by the caller)
    const int step_begin = wave * per;

    f32x4 acc[SLABS];
#pragma unroll
    for (int s = 0; s < SLABS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};

    // rows beyond N repeat the last row: their products only reach outputs that are never stored
    const bf16_t* w0[SLABS];
    const bf16_t* w1[SLABS];
#pragma unroll
    for (int s = 0; s < SLABS; ++s) {
        const int row = n_base + s * 16 + 2 * kg + (r >> 3);
        w0[s] = W + static_cast<int64_t>(min(row, N - 1)) * ldw + (r & 7) * 8;
        w1[s] = W + static_cast<int64_t>(min(row + 8, N - 1)) * ldw + (r & 7) * 8;
    }
    // after the exchange of halves, lane (q, i) holds row 2q + i/8 + 8 * (i/4 % 2) and k-group i % 4 of the step;
    // the operand's lane (kg, r) takes it from there
    const int source_lane = 16 * ((r >> 1) & 3) + 8 * (r & 1) + 4 * (r >> 3) + kg;
    const int xr = r % MP;
    const bool xok = xr < M;
    const int x_at = (r / MP) * 32 + kg * 8;
    const bf16_t* xrow = X + static_cast<int64_t>(xok ? xr : 0) * ldx + x_at;
    __shared__ float s_rstd[16];

    // Workgroups do not all walk K from the same end: every 64 of them start one group of steps later than the 64
    // before (and wrap around).  With everybody at the same offset of its rows at the same time the memory channels
    // are loaded unevenly; staggered like this the gate+up product of the 8B shape streams 6% faster (a stagger that
    // changes with every workgroup, or with every 8, is slower than none).  The order of a workgroup's sums depends on
    // its place in the grid only, so results stay the same from run to run and for any rows beside.
    const int groups = per / UNROLL;
    const int rot = static_cast<int>((blockIdx.x / STAGGER_BLOCKS) % static_cast<unsigned>(groups));

    // SCALED: 1 / sqrt(mean(x^2) + eps) of every row from the parts of its sum of squares, all rows at once:
    // THREADS / 16 threads a row, each with four 16-byte loads in flight first of all, so that one round trip to
    // memory brings rows of up to THREADS parts (any number of parts is taken; no multiple of four: one by one).
    constexpr int TPR = THREADS / 16;
    const int srow = tid / TPR, sl = tid % TPR;
    const bool sok = SCALED && srow < M;
    const float* src = SCALED ? scale.sumsq + static_cast<int64_t>(sok ? srow : 0) * scale.parts : nullptr;
    const int quads = (SCALED && (scale.parts & 3) == 0) ? scale.parts / 4 : 0;
    f32x4 first_parts[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        first_parts[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (sok && j * TPR + sl < quads) first_parts[j] = *reinterpret_cast<const f32x4*>(src + 4 * (j * TPR + sl));
    }

    for (int gi = 0; gi < groups; ++gi) {
        const int ks = step_begin + (gi + rot >= groups ? gi + rot - groups : gi + rot) * UNROLL;
        bf16x8 xb[UNROLL], wa[UNROLL][SLABS];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int pair_k = ((ks + u) & ~1) * 32;
#pragma unroll
            for (int s = 0; s < SLABS; ++s)
                wa[u][s] = __builtin_bit_cast(bf16x8, stream_load16(((u & 1) ? w1[s] : w0[s]) + pair_k));
            if (u % PACK == 0) {
                xb[u] = zeros8();
                if (xok) xb[u] = *reinterpret_cast<const bf16x8*>(xrow + (ks + u) * 32);
            }
        }
        if (SCALED && gi == 0) {
            // the parts' loads went out before this group's; adding them up here keeps their round trip to memory
            // beside the weights'.  The factors are read in the epilogue, behind the barrier that it needs anyway.
            float sum = 0.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) sum += (first_parts[j][0] + first_parts[j][1]) + (first_parts[j][2] + first_parts[j][3]);
            if (quads > 0) {
                for (int q0 = 4 * TPR; q0 < quads; q0 += 4 * TPR) {  // rows of more than 16 * TPR parts
                    f32x4 v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int q = q0 + j * TPR + sl;
                        v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                        if (sok && q < quads) v[j] = *reinterpret_cast<const f32x4*>(src + 4 * q);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) sum += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
                }
            } else {
                for (int p = sl; sok && p < scale.parts; p += TPR) sum += src[p];
            }
#pragma unroll
            for (int off = TPR / 2; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, TPR);
            if (sl == 0 && sok) s_rstd[srow] = 1.0f / sqrtf(sum / static_cast<float>(K) + scale.eps);
        }
        // every load of the group is on its way; now the lane exchanges
#pragma unroll
        for (int u = 0; u < UNROLL; u += 2) {
#pragma unroll
            for (int s = 0; s < SLABS; ++s) {
                const i32x4 l0 = __builtin_bit_cast(i32x4, wa[u][s]);
                const i32x4 l1 = __builtin_bit_cast(i32x4, wa[u + 1][s]);
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
                wa[u][s] = __builtin_bit_cast(bf16x8, a0);
                wa[u + 1][s] = __builtin_bit_cast(bf16x8, a1);
            }
        }
        if (PACK > 1) {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (u % PACK != 0) {
                    const i32x4 src = __builtin_bit_cast(i32x4, xb[u - u % PACK]);
                    i32x4 moved;
#pragma unroll
                    for (int e = 0; e < 4; ++e) moved[e] = row_shift_left(src[e], (u % PACK) * MP);
                    xb[u] = __builtin_bit_cast(bf16x8, moved);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int s = 0; s < SLABS; ++s)
                acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u][s], xb[u], acc[s], 0, 0, 0);
    }

#pragma unroll
    for (int s = 0; s < SLABS; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][s][4 * kg + i][r] = acc[s][i];
    __syncthreads();
    epilogue<SLABS, 1, KW, SWIGLU>(red, C, ldc, M, N, n_base, mode, tid, sumsq_out, parts_out,
                                   SCALED ? s_rstd : nullptr, copy_out, ldcopy, copy_scale);
}

template <int SLABS, int MT, int KW, bool SWIGLU>
void launch(bool xlds, const bf16_t* X, int64_t ldx, const bf16_t* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
            int K, int mode, hipStream_t stream) {
    const unsigned blocks = (N + SLABS * 16 - 1) / (SLABS * 16);
    const size_t red_bytes = sizeof(float) * KW * SLABS * MT * 16 * 17;
    if (MT == 1 && xlds) {
        const size_t x_bytes = static_cast<size_t>(K) * M * 2;
        hipLaunchKernelGGL((gemm_skinny_kernel<SLABS, 1, KW, SWIGLU, true>), dim3(blocks), dim3(KW * PULSE_WAVE),
                           x_bytes > red_bytes ? x_bytes : red_bytes, stream, X, ldx, W, ldw, C, ldc, M, N, K, mode);
    } else {
        hipLaunchKernelGGL((gemm_skinny_kernel<SLABS, MT, KW, SWIGLU, false>), dim3(blocks), dim3(KW * PULSE_WAVE),
                           red_bytes, stream, X, ldx, W, ldw, C, ldc, M, N, K, mode);
    }
}


template <int SLABS, int KW, bool SWIGLU>
void launch_stream(int pack, const bf16_t* X, int64_t ldx, const bf16_t* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                   int K, int mode, const RowScale& scale, float* sumsq_out, int parts_out, bf16_t* copy_out, int64_t ldcopy,
                   const bf16_t* copy_scale, hipStream_t stream) {
    const dim3 grid((N + SLABS * 16 - 1) / (SLABS * 16)), block(KW * PULSE_WAVE);
    const size_t red_bytes = sizeof(float) * KW * SLABS * 16 * 17;
#define PULSE_STREAM(P, SCALED)                                                                                          \
    hipLaunchKernelGGL((gemm_skinny_stream_kernel<SLABS, KW, P, SWIGLU, SCALED>), grid, block, red_bytes, stream, X, ldx, \
                       W, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy_out, ldcopy, copy_scale)
#define PULSE_STREAM_PACKS(SCALED)                    \
    do {                                              \
        if (pack == 8) PULSE_STREAM(8, SCALED);       \
        else if (pack == 4) PULSE_STREAM(4, SCALED);  \
        else if (pack == 2) PULSE_STREAM(2, SCALED);  \
        else PULSE_STREAM(1, SCALED);                 \
    } while (0)
    if (scale.sumsq) PULSE_STREAM_PACKS(true);
    else PULSE_STREAM_PACKS(false);
#undef PULSE_STREAM_PACKS
#undef PULSE_STREAM
}

// The most k-steps one load of X can serve for M rows.
int pack_for(int M) { return M <= 2 ? 8 : (M <= 4 ? 4 : (M <= 8 ? 2 : 1)); }

}  // namespace

// mode: 0 store bfloat16, 1 store float32, 2 add into float32.  swiglu != 0: W holds gate and up rows interleaved in
// slabs of 16 (gate slab, up slab, ...), N counts both, C is bfloat16 [M, N / 2] = silu(gate) * up.  tune: 0 lets the
// entry point choose the kernel.
// The same with the fusions of the streaming kernel (M <= 16, K a multiple of 1024), each optional:
//   scale_sumsq != null: row m of the product is multiplied by 1 / sqrt(sum(scale_sumsq[m, :]) / K + eps) before it is
//     stored (or goes through SwiGLU): the division of an RMSNorm, applied behind the product, from the sums of
//     squares [M, scale_parts] of the rows that were normed (any split of a row into parts); the norm's weight has to
//     be part of X already (see copy_scale);
//   sumsq_out != null (mode 2 only): besides adding into C, leave sumsq_out[row * parts + slab] = sum of squares of the
//     new values of C[row, 16 slab .. 16 slab + 15], parts = ceil(N / 16);
//   copy_out != null (mode 2 only): the new values of C once more as bfloat16, row stride ldcopy, each multiplied by
//     copy_scale[column] first (bfloat16 [N], the weight of the norm that reads C next; null: as they are).
// pulse_gemm_skinny_fusable says whether the streaming kernel takes a shape.
extern "C" int pulse_gemm_skinny_fusable(int M, int N, int K) { return M >= 1 && M <= 16 && N > 0 && K > 0 && K % 1024 == 0; }

extern "C" int pulse_gemm_skinny_fused(const void* X, int64_t ldx, const void* W, int64_t ldw, void* C, int64_t ldc, int M,
                                       int N, int K, int mode, int swiglu, int tune, const float* scale_sumsq,
                                       int scale_parts, float scale_eps, float* sumsq_out, void* copy_out,
                                       int64_t ldcopy, const void* copy_scale, hipStream_t stream) {
    const bool fused = scale_sumsq != nullptr || sumsq_out != nullptr || copy_out != nullptr;
    if (fused) {
        PULSE_REQUIRE(pulse_gemm_skinny_fusable(M, N, K) && tune != 9, "gemm_skinny: M=%d N=%d K=%d cannot take the fused kernel", M, N, K);
        PULSE_REQUIRE(sumsq_out == nullptr || (mode == OUT_ADD_F32 && !swiglu), "gemm_skinny: row sums of squares come with adding into float32 only");
        PULSE_REQUIRE(copy_out == nullptr || (mode == OUT_ADD_F32 && !swiglu && ldcopy >= N), "gemm_skinny: the bfloat16 copy comes with adding into float32 only");
        PULSE_REQUIRE(scale_sumsq == nullptr || (scale_parts > 0 && (reinterpret_cast<uintptr_t>(scale_sumsq) % 16) == 0),
                      "gemm_skinny: the row sums of squares need their number of parts and 16-byte alignment");
    }
    PULSE_REQUIRE(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: sizes M=%d (at most 64) N=%d K=%d", M, N, K);
    PULSE_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K,
                  "gemm_skinny: K and the row strides must be multiples of 8 (16-byte loads)");
    PULSE_REQUIRE((reinterpret_cast<uintptr_t>(X) % 16) == 0 && (reinterpret_cast<uintptr_t>(W) % 16) == 0,
                  "gemm_skinny: operands must be 16-byte aligned");
    PULSE_REQUIRE(mode >= 0 && mode <= 2, "gemm_skinny: unknown output mode %d", mode);
    PULSE_REQUIRE(X && W && C, "gemm_skinny: null pointer");
    if (swiglu) {
        PULSE_REQUIRE(N % 32 == 0 && mode == OUT_BF16 && ldc >= N / 2, "gemm_skinny: SwiGLU needs N %% 32 == 0 and bfloat16 output");
        PULSE_REQUIRE(M <= 32, "gemm_skinny: the SwiGLU epilogue takes at most 32 rows, got %d", M);
    } else {
        PULSE_REQUIRE(ldc >= N, "gemm_skinny: output row stride too small");
    }
    if (M == 0) return 0;
    const bf16_t* x = static_cast<const bf16_t*>(X);
    RowScale scale{scale_sumsq, scale_parts, scale_eps};
    const int parts_out = (N + 15) / 16;
    bf16_t* copy = static_cast<bf16_t*>(copy_out);
    const bf16_t* cscale = copy ? static_cast<const bf16_t*>(copy_scale) : nullptr;
    const bf16_t* w = static_cast<const bf16_t*>(W);
    const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    const int units = pulse_compute_units();
    const bool wide = N >= 64 * units;  // enough slabs that pairs of them still give every compute unit two workgroups
    // tune (tests and measurements): decimal digits S K P, S slabs (1, 2), K wavefronts (4, 8), P = 1 + log2 of the
    // k-steps a load of X serves (1..4), all for the streaming kernel; 9 asks for the general kernel.
    int t_slabs = 0, t_kw = 0, t_pack = 0;
    if (tune > 0 && tune != 9) {
        t_slabs = tune / 100, t_kw = tune / 10 % 10, t_pack = 1 << (tune % 10 - 1);
        PULSE_REQUIRE((t_slabs == 1 || t_slabs == 2) && (t_kw == 4 || t_kw == 8) && tune % 10 >= 1 && tune % 10 <= 4,
                      "gemm_skinny: unknown tuning %d", tune);
        PULSE_REQUIRE(mt == 1 && K % (256 * t_kw) == 0 && M <= 16 / t_pack && (!swiglu || t_slabs == 2),
                      "gemm_skinny: tuning %d does not fit M=%d K=%d", tune, M, K);
    }
    if (mt == 1 && tune != 9 && (t_kw ? true : K % 1024 == 0)) {
        // the streaming kernel: pairs of slabs when there are many (or, from 8 rows of X on, enough of them: a
        // pair shares its loads of X), else single slabs with more wavefronts along K
        // (also where single slabs would put two workgroups on some compute units and pairs one on each: 5,120
        // weight rows, o and down of the 14B shape, at 8 rows 16.2 -> 14.7 us and 44.7 -> 36.9 us)
        auto fullest = [&](int rows) { return ((N + rows - 1) / rows + units - 1) / units * rows; };   // weight rows on the fullest unit
        // (from 8 rows on, pairs also where they still reach three quarters of the units: N / 32 >= 3 units / 4)
        const bool pairs = swiglu || wide || (M >= 8 && (N >= 24 * units || fullest(16) >= fullest(32)));
        const int slabs = t_slabs ? t_slabs : (pairs ? 2 : 1);
        const int kw = t_kw ? t_kw : ((K % 2048 == 0 && !pairs) ? 8 : 4);
        const int pack = t_pack ? t_pack : pack_for(M);
        if (swiglu) {
            if (kw == 8) launch_stream<2, 8, true>(pack, x, ldx, w, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy, ldcopy, cscale, stream);
            else launch_stream<2, 4, true>(pack, x, ldx, w, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy, ldcopy, cscale, stream);
        } else if (slabs == 2) {
            if (kw == 8) launch_stream<2, 8, false>(pack, x, ldx, w, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy, ldcopy, cscale, stream);
            else launch_stream<2, 4, false>(pack, x, ldx, w, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy, ldcopy, cscale, stream);
        } else {
            if (kw == 8) launch_stream<1, 8, false>(pack, x, ldx, w, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy, ldcopy, cscale, stream);
            else launch_stream<1, 4, false>(pack, x, ldx, w, ldw, C, ldc, M, N, K, mode, scale, sumsq_out, parts_out, copy, ldcopy, cscale, stream);
        }
        PULSE_LAUNCH_CHECK("gemm_skinny");
        return 0;
    }
    PULSE_REQUIRE(!fused, "gemm_skinny: K=%d takes no fused kernel", K);
    // X goes through LDS when it is small enough for two workgroups a compute unit
    const bool xlds = mt == 1 && K % 32 == 0 && static_cast<size_t>(K) * M * 2 <= XLDS_BYTES;
    if (swiglu) {
        if (mt == 1) launch<2, 1, 4, true>(xlds, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else launch<2, 2, 8, true>(false, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
    } else if (mt == 1) {
        if (wide) launch<2, 1, 4, false>(xlds, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else launch<1, 1, 4, false>(xlds, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
    } else if (mt == 2) {
        if (wide) launch<2, 2, 8, false>(false, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else launch<1, 2, 8, false>(false, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
    } else {
        launch<1, 4, 8, false>(false, x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
    }
    PULSE_LAUNCH_CHECK("gemm_skinny");
    return 0;
}

extern "C" int pulse_gemm_skinny(const void* X, int64_t ldx, const void* W, int64_t ldw, void* C, int64_t ldc, int M,
                                 int N, int K, int mode, int swiglu, int tune, hipStream_t stream) {
    return pulse_gemm_skinny_fused(X, ldx, W, ldw, C, ldc, M, N, K, mode, swiglu, tune, nullptr, 0, 0.f, nullptr, nullptr, 0,
                                   nullptr, stream);
}
