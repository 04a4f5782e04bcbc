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

enum OutMode : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_ADD_F32 = 2 };

__device__ __forceinline__ bf16x8 zeros8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
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

    if (!SWIGLU) {
        for (int e = tid; e < TILES * 256; e += THREADS) {
            const int tile = e / 256;
            const int m_in = (e % 256) / 16;
            const int n_in = e % 16;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < KW; ++w) v += red[w][tile][n_in][m_in];
            const int m = (tile % MT) * 16 + m_in;
            const int n = n_base + (tile / MT) * 16 + n_in;
            if (m < M && n < N) {
                const int64_t at = static_cast<int64_t>(m) * ldc + n;
                if (mode == OUT_BF16) static_cast<bf16_t*>(C)[at] = f32_to_bf16(v);
                else if (mode == OUT_F32) static_cast<float*>(C)[at] = v;
                else static_cast<float*>(C)[at] += v;
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
            const int m = mt * 16 + m_in;
            const int n = n_base / 2 + pair * 16 + n_in;
            if (m < M && 2 * n < N) {  // N counts gate and up rows together
                const float v = g / (1.0f + expf(-g)) * u;
                static_cast<bf16_t*>(C)[static_cast<int64_t>(m) * ldc + n] = f32_to_bf16(v);
            }
        }
    }
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

}  // namespace

// mode: 0 store bfloat16, 1 store float32, 2 add into float32.  swiglu != 0: W holds gate and up rows interleaved in
// slabs of 16 (gate slab, up slab, ...), N counts both, C is bfloat16 [M, N / 2] = silu(gate) * up.
extern "C" int pulse_gemm_skinny(const void* X, int64_t ldx, const void* W, int64_t ldw, void* C, int64_t ldc, int M,
                                 int N, int K, int mode, int swiglu, hipStream_t stream) {
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
    const bf16_t* w = static_cast<const bf16_t*>(W);
    const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
    // X goes through LDS when it is small enough for two workgroups a compute unit
    const bool xlds = mt == 1 && K % 32 == 0 && static_cast<size_t>(K) * M * 2 <= XLDS_BYTES;
    const bool wide = N >= 16384;  // enough slabs that pairs of them still fill the chip
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
