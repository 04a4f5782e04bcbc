// C[M, N] = X[M, K] * W[N, K]^T in bfloat16 on the matrix cores for 17 to 64 rows and a weight of FEW rows (the
// projections into and out of attention, the feed-forward's way back): a weight of some thousand rows gives the chip
// one or two 16-row slabs a compute unit, and a wavefront that walks all of K for a slab alone is bound by its own
// latencies, not by the memory (6,144 weight rows at 64 rows of X: 2.4 TB/s).  Here a workgroup of four wavefronts
// owns ONE slab of 16 weight rows and all of K: the wavefronts walk K together in chunks of 256, each taking 64 k of
// every chunk (one whole 128-byte line of each weight row), so that four times as many wavefronts stream the weight,
// all four read the same chunk of X from LDS (a quarter of it each), and their partial sums meet in LDS in
// wavefront order.  Because the workgroup holds complete sums it can finish what the few-rows product finishes:
// add into the float32 residual, leave the new rows' sums of squares (16 columns a part) and a rounded copy with the
// next norm's weight multiplied in, and multiply its rows by 1 / sqrt(mean + eps) from such sums of its input
// (the RMSNorm moved behind the product): no shares of K go through memory, and no norm kernel adds them up.
//
// X goes through LDS once a workgroup, two stages, one barrier a chunk; the weight rows come straight into registers
// seven chunks ahead (14 KB a wavefront in flight), whole lines per 8 lanes, and are brought into the matrix-core
// layout with DPP and ds_bpermute as in the few-rows kernel.  Accumulation is float32
// (reference: cublasGemmEx with CUBLAS_COMPUTE_32F, src/ops/kernels/cuda/matmul_kernel.cu:132-154).
#include "common.h"

#include <math.h>

#include <utility>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int KC = 256;        // k of a chunk: 64 for each of the four wavefronts
constexpr int KW = 4;          // wavefronts that share K out among themselves
constexpr int RING = 8;        // register sets of weight chunks: loads run RING - 1 chunks ahead
constexpr int XD = 2;          // register sets of chunks of X: its loads (from L2 mostly) run XD chunks ahead
static_assert(RING % XD == 0, "a chunk's number modulo RING names its set of X too");
constexpr int XROW = KC + 8;   // bfloat16 a row of X takes in LDS: 16 bytes of padding spread the rows over the banks

enum RowsMode : int { ROWS_BF16 = 0, ROWS_ADD_F32 = 2 };

template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

struct RowsArgs {
    const bf16_t* X; int64_t ldx;
    const bf16_t* W; int64_t ldw;
    void* C; int64_t ldc;
    int M, N, K, mode;
    const float* scale_sumsq; int scale_parts; float scale_eps;   // rows of the result times 1 / sqrt(sum / K + eps)
    float* sumsq_out; int parts_out;                               // [M, N / 16]
    bf16_t* copy_out; int64_t ldcopy; const bf16_t* copy_scale;    // bfloat16(new C * copy_scale[column])
};

// MT tiles of 16 rows of X; SL slabs of 16 weight rows a workgroup, KW wavefronts each.  Every workgroup fetches all
// of X (from L2): the fewer workgroups, the less of that traffic, which is what bounds a workgroup a slab (6,144
// weight rows at 64 rows of X: 384 workgroups move 200 MB of X for 50 MB of weight).
template <int MT, int SL>
__global__ __launch_bounds__(SL* KW* PULSE_WAVE) void gemm_rows_kernel(RowsArgs a) {
    constexpr int NW = SL * KW;
    constexpr int THREADS = NW * PULSE_WAVE;
    __shared__ __attribute__((aligned(16))) bf16_t s_x[2][16 * MT * XROW];
    __shared__ float s_rstd[16 * MT];
    static_assert(sizeof(f32x4) * NW * MT * PULSE_WAVE <= sizeof(bf16_t) * 2 * 16 * MT * XROW,
                  "the wavefronts' partial sums take the place of the stages of X at the end");
    constexpr int ROWP = KC / 8;                   // 16-byte pieces of a row of a chunk of X
    constexpr int PIECES = 16 * MT * ROWP;
    constexpr int XP = PIECES / THREADS;           // pieces a thread stages (2 MT)
    static_assert(PIECES % THREADS == 0, "every thread stages the same number of pieces");

    const int tid = threadIdx.x;
    const int wave_all = tid / PULSE_WAVE;
    const int slab = wave_all / KW;     // which of the workgroup's slabs
    const int wave = wave_all % KW;     // which 64 k of every chunk
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;
    const int n_base = (blockIdx.x * SL + slab) * 16;
    const int M = a.M, N = a.N;
    const int chunks = a.K / KC;
    // Workgroups do not all walk K from the same end (which loads the memory channels unevenly): the owners of every
    // four slabs start a chunk later than the owners of the four before, and wrap around.  The order of a column's
    // sums depends on the column and K only, not on how many slabs a workgroup holds (1, 2 or 4: the four are its own
    // or its neighbours').
    const int rot = static_cast<int>((blockIdx.x * SL / 4) % static_cast<unsigned>(chunks));
    auto placed = [&](int c) { return c + rot >= chunks ? c + rot - chunks : c + rot; };

    // Weight loads: 8 consecutive lanes fetch one whole 128-byte line (row 2kg + r/8, piece r%8 of this wavefront's
    // 64 k of the chunk), the second load the rows 8 further on.
    const int wrow = n_base + 2 * kg + (r >> 3);
    const bf16_t* w0 = a.W + static_cast<int64_t>(min(wrow, N - 1)) * a.ldw + wave * 64 + (r & 7) * 8;
    const bf16_t* w1 = a.W + static_cast<int64_t>(min(wrow + 8, N - 1)) * a.ldw + wave * 64 + (r & 7) * 8;
    const int source_lane = 16 * ((r >> 1) & 3) + 8 * (r & 1) + 4 * (r >> 3) + kg;

    // X pieces of a chunk that this thread stages: piece p = tid + THREADS i is row p / ROWP, columns 8 (p % ROWP)..
    // Every load of the walk is issued whatever the row or the chunk (a load under a condition would keep the
    // compiler from counting the loads in flight): rows beyond M repeat row M - 1, whose products only reach outputs
    // that are never stored, and chunks beyond the last one fetch the last one again.
    const bf16_t* xsrc[XP];
    int xdst[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int p = tid + THREADS * i;
        const int xr = p / ROWP, xc = p % ROWP;
        xsrc[i] = a.X + static_cast<int64_t>(min(xr, M - 1)) * a.ldx + xc * 8;
        xdst[i] = xr * XROW + xc * 8;
    }

    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    bf16x8 xg[XD][XP];
    bf16x8 wr[RING][2];
    auto load_x = [&](int c, bf16x8 (&x)[XP]) {
        const int64_t at = static_cast<int64_t>(placed(min(c, chunks - 1))) * KC;
#pragma unroll
        for (int i = 0; i < XP; ++i) x[i] = *reinterpret_cast<const bf16x8*>(xsrc[i] + at);
    };
    auto load_w = [&](int c, bf16x8 (&w)[2]) {
        const int64_t at = static_cast<int64_t>(placed(min(c, chunks - 1))) * KC;
        w[0] = __builtin_bit_cast(bf16x8, stream_load16(w0 + at));
        w[1] = __builtin_bit_cast(bf16x8, stream_load16(w1 + at));
    };
    auto body = [&](auto J, int c) {
        constexpr int j = decltype(J)::value;
        bf16_t* stage = s_x[c & 1];
#pragma unroll
        for (int i = 0; i < XP; ++i) *reinterpret_cast<bf16x8*>(stage + xdst[i]) = xg[j % XD][i];
        // Everybody has left the chunk before the last one (they passed the barrier of the last one), whose stage
        // this is; after this barrier everybody sees this chunk.
        __syncthreads();
        load_x(c + XD, xg[j % XD]);
        load_w(c + RING - 1, wr[(j + RING - 1) % RING]);
        const i32x4 l0 = __builtin_bit_cast(i32x4, wr[j][0]);
        const i32x4 l1 = __builtin_bit_cast(i32x4, wr[j][1]);
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
            const bf16x8 wa = __builtin_bit_cast(bf16x8, h == 0 ? a0 : a1);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const bf16x8 xb = *reinterpret_cast<const bf16x8*>(stage + (16 * mt + r) * XROW + wave * 64 + h * 32 + kg * 8);
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb, acc[mt], 0, 0, 0);
            }
        }
    };

    load_x(0, xg[0]);
    load_w(0, wr[0]);
    static_for<XD - 1>([&](auto J) { load_x(decltype(J)::value + 1, xg[decltype(J)::value + 1]); });
    static_for<RING - 2>([&](auto J) { load_w(decltype(J)::value + 1, wr[decltype(J)::value + 1]); });
    // 1 / sqrt(mean(x^2) + eps) of every row of X from the parts of its sum of squares: four threads a row, in a
    // fixed order; asked for behind the first weights, read in the epilogue behind its barrier.
    if (a.scale_sumsq && tid < 4 * 16 * MT) {
        const int row = tid / 4, sl = tid % 4;
        float sum = 0.f;
        if (row < M) {
            const float* src = a.scale_sumsq + static_cast<int64_t>(row) * a.scale_parts;
            const int quads = (a.scale_parts & 3) == 0 ? a.scale_parts / 4 : 0;
            for (int q = sl; q < quads; q += 4) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(src + 4 * q);
                sum += (v[0] + v[1]) + (v[2] + v[3]);
            }
            for (int p = 4 * quads + sl; p < a.scale_parts; p += 4) sum += src[p];
        }
        sum += __shfl_xor(sum, 1, 4);
        sum += __shfl_xor(sum, 2, 4);
        if (sl == 0 && row < 16 * MT) s_rstd[row] = row < M ? 1.0f / sqrtf(sum / static_cast<float>(a.K) + a.scale_eps) : 0.f;
    }
    int c = 0;
    for (; c + RING <= chunks; c += RING)   // whole turns of the ring without a branch inside
        static_for<RING>([&](auto J) { body(J, c + decltype(J)::value); });
    static_for<RING - 1>([&](auto J) {
        if (c + decltype(J)::value < chunks) body(J, c + decltype(J)::value);
    });

    // The four wavefronts' sums meet in the memory of the stages, which everybody has left after a barrier; then
    // wavefront w finishes row tiles w, w + 4, ..: lane (kg, r) holds columns n_base + 4 kg + i of row 16 mt + r.
    f32x4 (*s_red)[MT][PULSE_WAVE] = reinterpret_cast<f32x4 (*)[MT][PULSE_WAVE]>(&s_x[0][0]);
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) s_red[wave_all][mt][lane] = acc[mt];
    __syncthreads();
    const int n = n_base + 4 * kg;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        if (mt % KW != wave) continue;
        const int m = 16 * mt + r;
        f32x4 v = s_red[slab * KW][mt][lane];
#pragma unroll
        for (int w = 1; w < KW; ++w) v += s_red[slab * KW + w][mt][lane];   // in wavefront order
        if (a.scale_sumsq) v *= s_rstd[m];
        float sq = 0.f;
        if (m < M && n < N) {
            if (a.mode == ROWS_BF16) {
                bf16x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i] = (__bf16)v[i];
                *reinterpret_cast<bf16x4*>(static_cast<bf16_t*>(a.C) + static_cast<int64_t>(m) * a.ldc + n) = o;
            } else {
                float* dst = static_cast<float*>(a.C) + static_cast<int64_t>(m) * a.ldc + n;
                const f32x4 updated = *reinterpret_cast<const f32x4*>(dst) + v;
                *reinterpret_cast<f32x4*>(dst) = updated;
                sq = (updated[0] * updated[0] + updated[1] * updated[1]) + (updated[2] * updated[2] + updated[3] * updated[3]);
                if (a.copy_out) {
                    bf16x4 o;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        o[i] = (__bf16)(a.copy_scale ? updated[i] * bf16_to_f32(a.copy_scale[n + i]) : updated[i]);
                    *reinterpret_cast<bf16x4*>(a.copy_out + static_cast<int64_t>(m) * a.ldcopy + n) = o;
                }
            }
        }
        if (a.sumsq_out) {   // the four lanes of a row hold its 16 columns
            sq += __shfl_xor(sq, 16, PULSE_WAVE);
            sq += __shfl_xor(sq, 32, PULSE_WAVE);
            if (kg == 0 && m < M && n_base < N) a.sumsq_out[static_cast<int64_t>(m) * a.parts_out + n_base / 16] = sq;
        }
    }
}

}  // namespace

template <int MT>
void launch_rows_kernel(const RowsArgs& a, int slabs, hipStream_t stream) {
    const int groups = (a.N / 16 + slabs - 1) / slabs;
    if (slabs == 1) hipLaunchKernelGGL((gemm_rows_kernel<MT, 1>), dim3(groups), dim3(KW * PULSE_WAVE), 0, stream, a);
    else if (slabs == 2) hipLaunchKernelGGL((gemm_rows_kernel<MT, 2>), dim3(groups), dim3(2 * KW * PULSE_WAVE), 0, stream, a);
    else hipLaunchKernelGGL((gemm_rows_kernel<MT, 4>), dim3(groups), dim3(4 * KW * PULSE_WAVE), 0, stream, a);
}

// Whether pulse_gemm_rows takes a shape: 1..64 rows, whole 16-row slabs of the weight, K in chunks of 256.
extern "C" int pulse_gemm_rows_takes(int M, int N, int K) {
    return M >= 1 && M <= 64 && N > 0 && N % 16 == 0 && K > 0 && K % KC == 0;
}

// mode 0: C is bfloat16 [M, N].  mode 2: C is float32 [M, N] and the product is added to it; then
//   sumsq_out != null: sumsq_out[row * (N / 16) + slab] = sum of squares of the slab's 16 new values of the row;
//   copy_out != null: the new values of C once more as bfloat16 (row stride ldcopy), each multiplied by
//     copy_scale[column] first (bfloat16 [N], the weight of the norm that reads C next; null: as they are).
// slabs: see below.
// scale_sumsq != null (either mode): row m of the product is multiplied by 1 / sqrt(sum(scale_sumsq[m, :]) / K + eps)
//   before anything else is done with it (scale_sumsq float32 [M, scale_parts]: the sums of squares, in parts, of the
//   rows whose RMSNorm X stands for; the norm's weight must be part of X already).
extern "C" int pulse_gemm_rows(const void* X, int64_t ldx, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N,
                               int K, int mode, const float* scale_sumsq, int scale_parts, float scale_eps,
                               float* sumsq_out, void* copy_out, int64_t ldcopy, const void* copy_scale, int slabs,
                               hipStream_t stream) {
    PULSE_REQUIRE(pulse_gemm_rows_takes(M, N, K), "gemm_rows: M=%d (1..64) N=%d (a multiple of 16) K=%d (a multiple of %d)",
                  M, N, K, KC);
    PULSE_REQUIRE(X && W && C, "gemm_rows: null pointer");
    PULSE_REQUIRE(ldx % 8 == 0 && ldw % 8 == 0 && ldx >= K && ldw >= K, "gemm_rows: the row strides must be multiples of 8 and cover K");
    PULSE_REQUIRE((reinterpret_cast<uintptr_t>(X) % 16) == 0 && (reinterpret_cast<uintptr_t>(W) % 16) == 0 &&
                  (reinterpret_cast<uintptr_t>(C) % 16) == 0, "gemm_rows: operands must be 16-byte aligned");
    PULSE_REQUIRE(mode == ROWS_BF16 || mode == ROWS_ADD_F32, "gemm_rows: unknown output mode %d", mode);
    PULSE_REQUIRE(ldc % 4 == 0 && ldc >= N, "gemm_rows: the output's row stride must be a multiple of 4 and cover N");
    PULSE_REQUIRE((sumsq_out == nullptr && copy_out == nullptr) || mode == ROWS_ADD_F32,
                  "gemm_rows: sums of squares and the bfloat16 copy come with adding into float32 only");
    PULSE_REQUIRE(copy_out == nullptr || (ldcopy % 4 == 0 && ldcopy >= N && (reinterpret_cast<uintptr_t>(copy_out) % 8) == 0),
                  "gemm_rows: the copy's row stride must be a multiple of 4 and cover N");
    PULSE_REQUIRE(copy_scale == nullptr || copy_out != nullptr, "gemm_rows: copy_scale comes with copy_out");
    PULSE_REQUIRE(scale_sumsq == nullptr || (scale_parts > 0 && (reinterpret_cast<uintptr_t>(scale_sumsq) % 16) == 0),
                  "gemm_rows: the row sums of squares must be 16-byte aligned and have parts");
    RowsArgs a;
    a.X = static_cast<const bf16_t*>(X); a.ldx = ldx;
    a.W = static_cast<const bf16_t*>(W); a.ldw = ldw;
    a.C = C; a.ldc = ldc; a.M = M; a.N = N; a.K = K; a.mode = mode;
    a.scale_sumsq = scale_sumsq; a.scale_parts = scale_parts; a.scale_eps = scale_eps;
    a.sumsq_out = sumsq_out; a.parts_out = N / 16;
    a.copy_out = static_cast<bf16_t*>(copy_out); a.ldcopy = ldcopy; a.copy_scale = static_cast<const bf16_t*>(copy_scale);
    // slabs: 16-row slabs of the weight a workgroup (1, 2 or 4; 0 lets the entry point choose): a workgroup fetches
    // all of X, so few workgroups are better as long as they keep the memory busy
    if (slabs == 0) slabs = 2;
    PULSE_REQUIRE(slabs == 1 || slabs == 2 || slabs == 4, "gemm_rows: 1, 2 or 4 slabs a workgroup, got %d", slabs);
    if (M <= 32) launch_rows_kernel<2>(a, slabs, stream);
    else launch_rows_kernel<4>(a, slabs, stream);
    PULSE_LAUNCH_CHECK("gemm_rows");
    return 0;
}
