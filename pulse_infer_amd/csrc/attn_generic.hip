// Paged causal attention for any head size, page size and storage type: one
// wavefront per (token, query head), float32 arithmetic throughout.
//
// A token at position p sees keys lo..p of its own request through the block
// table, lo = max(0, p - window + 1) when a window is set, else 0.  Keys are
// taken 64 at a time (one per lane); the softmax is the running-maximum form
// (reference: src/ops/kernels/cuda/paged_attention.cu:88-137), the scale is a
// parameter (the reference fixes rsqrt(head_size), paged_attention.cu:108), and
// query head h reads kv head h / (nq / nkv) (paged_attention.cu:61-70).
//
// This is the kernel of the true 32-bit path and the fallback for sizes that the
// matrix-core kernels refuse.
#include "common.h"

#include <math.h>

namespace {

constexpr int MAX_ACC = 8;  // head_dim <= 512

struct AttnArgs {
    int nq, nkv, d;
    int64_t q_stride, o_stride;
    int page_size, num_pages, bt_width;
    float scale;
    int window;  // 0: all keys
};

template <typename TX, typename TC>
__global__ __launch_bounds__(64) void attn_generic_kernel(const TX* __restrict__ q, TX* __restrict__ out,
                                                          const TC* __restrict__ kcache,
                                                          const TC* __restrict__ vcache,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ token_entry,
                                                          const int* __restrict__ block_table, AttnArgs a) {
    extern __shared__ long long lds[];
    long long* v_s = lds;                                         // [64] value offsets of a tile's keys
    float* p_s = reinterpret_cast<float*>(lds + PULSE_WAVE);      // [64] a tile's probabilities
    float* q_s = p_s + PULSE_WAVE;                                // [d]  the scaled query

    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int d = a.d;
    const int group = a.nq / a.nkv;
    const int kvh = h / group;
    const int pos = positions[t];
    const int* bt = block_table + static_cast<int64_t>(token_entry[t]) * a.bt_width;
    const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;

    const TX* qrow = q + static_cast<int64_t>(t) * a.q_stride + static_cast<int64_t>(h) * d;
    for (int e = lane; e < d; e += PULSE_WAVE) q_s[e] = to_f32<TX>(qrow[e]) * a.scale;
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[MAX_ACC];
#pragma unroll
    for (int r = 0; r < MAX_ACC; ++r) acc[r] = 0.f;

    for (int j0 = lo; j0 <= pos; j0 += PULSE_WAVE) {
        const int j = j0 + lane;
        float s = -INFINITY;
        long long vbase = -1;
        if (j <= pos) {
            const int pi = j / a.page_size;
            const int page = pi < a.bt_width ? bt[pi] : -1;
            if (page >= 0 && page < a.num_pages) {
                const int slot = j % a.page_size;
                const int64_t pg = static_cast<int64_t>(page) * a.nkv + kvh;
                const TC* krow = kcache + (pg * a.page_size + slot) * d;
                float dot = 0.f;
                for (int e = 0; e < d; ++e) dot = fmaf(q_s[e], to_f32<TC>(krow[e]), dot);
                s = dot;
                vbase = pg * d * a.page_size + slot;
            }
        }
        const float tile_max = wave_max(s);
        const float m_new = fmaxf(m, tile_max);
        // every tile holds at least key j0 <= pos; were its page missing, m_new could still be -inf
        const float alpha = (m_new == -INFINITY) ? 1.f : expf(m - m_new);
        const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
        l = l * alpha + wave_sum(p);
        m = m_new;
        p_s[lane] = p;
        v_s[lane] = vbase;
        __syncthreads();
        const int nkeys = min(PULSE_WAVE, pos - j0 + 1);
#pragma unroll
        for (int r = 0; r < MAX_ACC; ++r) {
            const int e = lane + r * PULSE_WAVE;
            if (e < d) {
                float sum = 0.f;
                for (int jj = 0; jj < nkeys; ++jj) {
                    const long long vb = v_s[jj];
                    if (vb >= 0) sum = fmaf(p_s[jj], to_f32<TC>(vcache[vb + static_cast<int64_t>(e) * a.page_size]), sum);
                }
                acc[r] = acc[r] * alpha + sum;
            }
        }
        __syncthreads();
    }

    TX* orow = out + static_cast<int64_t>(t) * a.o_stride + static_cast<int64_t>(h) * d;
    const float inv_l = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int r = 0; r < MAX_ACC; ++r) {
        const int e = lane + r * PULSE_WAVE;
        if (e < d) orow[e] = from_f32<TX>(acc[r] * inv_l);
    }
}

}  // namespace

extern "C" int pulse_attn_generic(const void* q, int64_t q_stride, void* out, int64_t o_stride, int x_dtype,
                                  const void* kcache, const void* vcache, int c_dtype, const int* positions,
                                  const int* token_entry, const int* block_table, int bt_width, int tokens, int nq,
                                  int nkv, int d, int page_size, int num_pages, float scale, int window,
                                  hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && nq > 0 && nkv > 0 && d > 0, "attn_generic: bad sizes");
    PULSE_REQUIRE(nq % nkv == 0, "attn_generic: %d query heads are not a multiple of %d kv heads", nq, nkv);
    PULSE_REQUIRE(d <= PULSE_WAVE * MAX_ACC, "attn_generic: head_dim %d exceeds %d", d, PULSE_WAVE * MAX_ACC);
    PULSE_REQUIRE(nq < 65536, "attn_generic: at most 65535 query heads, got %d", nq);
    PULSE_REQUIRE(page_size > 0 && num_pages > 0 && bt_width > 0, "attn_generic: bad cache geometry");
    PULSE_REQUIRE(window >= 0, "attn_generic: negative window");
    PULSE_REQUIRE(q_stride >= static_cast<int64_t>(nq) * d && o_stride >= static_cast<int64_t>(nq) * d,
                  "attn_generic: row strides too small");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(c_dtype), "attn_generic: bad dtype tag");
    PULSE_REQUIRE(q && out && kcache && vcache && positions && token_entry && block_table, "attn_generic: null pointer");
    if (tokens == 0) return 0;
    AttnArgs a;
    a.nq = nq; a.nkv = nkv; a.d = d; a.q_stride = q_stride; a.o_stride = o_stride;
    a.page_size = page_size; a.num_pages = num_pages; a.bt_width = bt_width; a.scale = scale; a.window = window;
    const size_t lds = static_cast<size_t>(d) * sizeof(float) + PULSE_WAVE * sizeof(float) + PULSE_WAVE * sizeof(long long);
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        hipLaunchKernelGGL((attn_generic_kernel<TX, TC>), dim3(tokens, nq), dim3(64), lds, stream,
                           static_cast<const TX*>(q), static_cast<TX*>(out), static_cast<const TC*>(kcache),
                           static_cast<const TC*>(vcache), positions, token_entry, block_table, a)));
    PULSE_LAUNCH_CHECK("attn_generic");
    return 0;
}
