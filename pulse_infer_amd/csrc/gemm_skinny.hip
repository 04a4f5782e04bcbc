// C[M, N] = X[M, K] * W[N, K]^T for few rows (M <= 64) in bfloat16 on the matrix
// cores: the regime of decoding, where the product only has to stream the
// weight from HBM once.
//
// A workgroup of eight wavefronts owns SLABS slabs of 16 weight rows.  Each
// wavefront takes one eighth of K and runs v_mfma_f32_16x16x32_bf16 with the
// weight slab as the row operand and X^T as the column operand (both are 16-byte
// loads of 8 consecutive k), so the result is C^T: lane l holds output features
// 4*(l/16)+i of row l%16.  The eight partial tiles are summed through LDS in
// wavefront order, so the result is the same from run to run.  The epilogue
// stores bfloat16 or float32, adds into a float32 matrix (the residual), or
// applies SwiGLU to a (gate, up) pair of slabs of a slab-interleaved weight.
// Accumulation is float32 (reference: cublasGemmEx with CUBLAS_COMPUTE_32F,
// src/ops/kernels/cuda/matmul_kernel.cu:132-154).
#include "common.h"

#include <math.h>

namespace {

constexpr int KWAVES = 8;
constexpr int UNROLL = 8;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum OutMode : int { OUT_BF16 = 0, OUT_F32 = 1, OUT_ADD_F32 = 2 };

__device__ __forceinline__ bf16x8 zeros8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
}

template <int SLABS, int MT, bool SWIGLU>
__global__ __launch_bounds__(KWAVES* PULSE_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ X, int64_t ldx,
                                                                          const bf16_t* __restrict__ W, int64_t ldw,
                                                                          void* __restrict__ C, int64_t ldc, int M,
                                                                          int N, int K, int mode) {
    constexpr int TILES = SLABS * MT;
    __shared__ float red[KWAVES][TILES][16][17];

    const int tid = threadIdx.x;
    const int wave = tid / PULSE_WAVE;
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;
    const int n_base = blockIdx.x * SLABS * 16;

    const int steps = (K + 31) / 32;
    const int per = (steps + KWAVES - 1) / KWAVES;
    const int step_begin = wave * per;
    const int step_end = min(steps, step_begin + per);

    f32x4 acc[SLABS][MT];
#pragma unroll
    for (int s = 0; s < SLABS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[s][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const bf16_t* wrow[SLABS];
    bool wok[SLABS];
#pragma unroll
    for (int s = 0; s < SLABS; ++s) {
        const int n = n_base + s * 16 + r;
        wok[s] = n < N;
        wrow[s] = W + static_cast<int64_t>(wok[s] ? n : 0) * ldw;
    }
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        xok[mt] = m < M;
        xrow[mt] = X + static_cast<int64_t>(xok[mt] ? m : 0) * ldx;
    }

    // UNROLL k-steps at a time: all their loads are issued before the first product waits for one
    for (int ks = step_begin; ks < step_end; ks += UNROLL) {
        bf16x8 xb[UNROLL][MT], wa[UNROLL][SLABS];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k = (ks + u) * 32 + kg * 8;
            const bool kok = (ks + u < step_end) && k < K;
            const int kc = kok ? k : 0;  // always a valid address; what lies beyond K is zeroed below
            // rows beyond N or M read row 0: their products only reach outputs that are never stored
#pragma unroll
            for (int s = 0; s < SLABS; ++s) {
                wa[u][s] = *reinterpret_cast<const bf16x8*>(wrow[s] + kc);
                if (!kok) wa[u][s] = zeros8();
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xb[u][mt] = *reinterpret_cast<const bf16x8*>(xrow[mt] + kc);
                if (!kok) xb[u][mt] = zeros8();
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

#pragma unroll
    for (int s = 0; s < SLABS; ++s)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][s * MT + mt][4 * kg + i][r] = acc[s][mt][i];
    __syncthreads();

    if (!SWIGLU) {
        for (int e = tid; e < TILES * 256; e += KWAVES * PULSE_WAVE) {
            const int tile = e / 256;
            const int m_in = (e % 256) / 16;
            const int n_in = e % 16;
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < KWAVES; ++w) v += red[w][tile][n_in][m_in];
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
        for (int e = tid; e < PAIRS * MT * 256; e += KWAVES * PULSE_WAVE) {
            const int pt = e / 256;  // pair * MT + mt
            const int m_in = (e % 256) / 16;
            const int n_in = e % 16;
            const int pair = pt / MT, mt = pt % MT;
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int w = 0; w < KWAVES; ++w) {
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

template <int SLABS, int MT, bool SWIGLU>
void launch(const bf16_t* X, int64_t ldx, const bf16_t* W, int64_t ldw, void* C, int64_t ldc, int M, int N, int K,
            int mode, hipStream_t stream) {
    const unsigned blocks = (N + SLABS * 16 - 1) / (SLABS * 16);
    hipLaunchKernelGGL((gemm_skinny_kernel<SLABS, MT, SWIGLU>), dim3(blocks), dim3(KWAVES * PULSE_WAVE), 0, stream, X,
                       ldx, W, ldw, C, ldc, M, N, K, mode);
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
    // more slabs per workgroup reuse X better; fewer give more workgroups.  Aim for at least 512 workgroups.
    const int slabs_total = (N + 15) / 16;
    int slabs = 4 / mt;
    while (slabs > 1 && slabs_total / slabs < 512) slabs /= 2;
    if (swiglu && slabs < 2) slabs = 2;
    if (swiglu) {
        if (mt == 1 && slabs == 4) launch<4, 1, true>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else if (mt == 1) launch<2, 1, true>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else launch<2, 2, true>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
    } else {
        if (mt == 1 && slabs == 4) launch<4, 1, false>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else if (mt == 1 && slabs == 2) launch<2, 1, false>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else if (mt == 1) launch<1, 1, false>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else if (mt == 2 && slabs == 2) launch<2, 2, false>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else if (mt == 2) launch<1, 2, false>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
        else launch<1, 4, false>(x, ldx, w, ldw, C, ldc, M, N, K, mode, stream);
    }
    PULSE_LAUNCH_CHECK("gemm_skinny");
    return 0;
}
