// C[M, N] = A[M, K] * W[N, K]^T with float32 multiply-adds in a fixed order.
//
// This is the matrix product of the true 32-bit path: no matrix-core
// instruction and no reduced-precision mode is involved, every product and sum
// is an IEEE float32 fma.  Each output element is accumulated over k = 0..K-1 in
// ascending order whatever M is, so a row's result does not depend on what else
// is in the batch.  Inputs may be stored as bfloat16 (they are widened exactly).
// (reference: cublasSgemm, src/ops/kernels/cuda/matmul_kernel.cu:70-88)
#include "common.h"

namespace {

constexpr int BM = 64;
constexpr int BN = 64;
constexpr int BK = 16;
constexpr int TM = 4;
constexpr int TN = 4;

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                       TC* __restrict__ C, int M, int N, int K,
                                                       int64_t lda, int64_t ldw, int64_t ldc) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16;  // column group
    const int ty = tid / 16;  // row group
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN;

    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

    // each thread stages 4 elements of A and 4 of W per k-step: row = tid / 4, k = (tid % 4) * 4 + e
    const int lrow = tid / 4;
    const int lk = (tid % 4) * 4;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int m = m0 + lrow;
            const int n = n0 + lrow;
            As[lk + e][lrow] = (m < M && k < K) ? to_f32<TA>(A[static_cast<int64_t>(m) * lda + k]) : 0.f;
            Ws[lk + e][lrow] = (n < N && k < K) ? to_f32<TW>(W[static_cast<int64_t>(n) * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = As[kk][ty * TM + i];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = Ws[kk][tx * TN + j];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + ty * TM + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + tx * TN + j;
            if (n < N) C[static_cast<int64_t>(m) * ldc + n] = from_f32<TC>(acc[i][j]);
        }
    }
}

}  // namespace

extern "C" int pulse_gemm_f32(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype,
                              int M, int N, int K, int64_t lda, int64_t ldw, int64_t ldc, hipStream_t stream) {
    PULSE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
    PULSE_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: leading dimensions too small");
    PULSE_REQUIRE(pulse_dtype_ok(a_dtype) && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(c_dtype), "gemm_f32: bad dtype tag");
    PULSE_REQUIRE(A && W && C, "gemm_f32: null pointer");
    if (M == 0) return 0;
    const unsigned gx = (N + BN - 1) / BN, gy = (M + BM - 1) / BM;
    PULSE_REQUIRE(gy < 65536, "gemm_f32: M=%d is too large for one launch", M);
    PULSE_DISPATCH_DTYPE(a_dtype, TA, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        hipLaunchKernelGGL((gemm_f32_kernel<TA, TW, TC>), dim3(gx, gy), dim3(256), 0, stream,
                           static_cast<const TA*>(A), static_cast<const TW*>(W), static_cast<TC*>(C), M, N, K,
                           lda, ldw, ldc))));
    PULSE_LAUNCH_CHECK("gemm_f32");
    return 0;
}
