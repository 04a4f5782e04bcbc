// One pass over the fused projection output of a step: per-head RMSNorm of q
// and k, rotation of q and k by the position table, q written back in place,
// k and v written into their cache pages.
//
// Cache layout per (page, kv head): K is [page_size, head_dim] (a key's
// elements contiguous), V is [head_dim, page_size] (a channel's keys
// contiguous), which is what the attention kernels' matrix-core operands want.
//
// Replaces five launches of the reference (q_norm, k_norm, two rotations, the
// page write: src/model/qwen3/model.cpp:815-848; formulas
// src/ops/kernels/cuda/rmsnorm_kernel.cu:97-157, rope_kernel.cu:76-132,
// paged_kv_write.cu:31-52).  Norm and rotation are float32 with one rounding.
#include "common.h"

namespace {

constexpr int MAX_PAIRS_PER_LANE = 4;  // head_dim <= 512

struct QkRopeArgs {
    int nq, nkv, d;
    int64_t row_stride;
    float eps;
    int rotary_dim;  // 0: no rotation
    int pairing;     // 0: (2i, 2i+1)   1: (i, i + rotary_dim/2)
    int page_size, num_pages, bt_width;
    int write_kv;
};

template <typename TX, typename TW, typename TC>
__global__ __launch_bounds__(64) void qk_rope_kv_kernel(TX* __restrict__ qkv, const TW* __restrict__ q_w,
                                                        const TW* __restrict__ k_w, const float* __restrict__ cos_t,
                                                        const float* __restrict__ sin_t, TC* __restrict__ kcache,
                                                        TC* __restrict__ vcache, const int* __restrict__ positions,
                                                        const int* __restrict__ token_entry,
                                                        const int* __restrict__ block_table, QkRopeArgs a) {
    const int t = blockIdx.x;
    const int hh = blockIdx.y;
    const int lane = threadIdx.x;
    const int d = a.d;
    const int half_rot = a.rotary_dim / 2;
    const bool is_q = hh < a.nq;
    const int g = hh - a.nq;
    TX* row = qkv + static_cast<int64_t>(t) * a.row_stride;
    TX* x = is_q ? row + static_cast<int64_t>(hh) * d : row + static_cast<int64_t>(a.nq + g) * d;
    const TW* w = is_q ? q_w : k_w;

    int ia[MAX_PAIRS_PER_LANE], ib[MAX_PAIRS_PER_LANE];
    float xa[MAX_PAIRS_PER_LANE], xb[MAX_PAIRS_PER_LANE];
    float ss = 0.f;
    const int npairs = d / 2;
#pragma unroll
    for (int r = 0; r < MAX_PAIRS_PER_LANE; ++r) {
        const int p = lane + r * PULSE_WAVE;
        if (p < npairs) {
            if (p < half_rot) {
                ia[r] = a.pairing == 0 ? 2 * p : p;
                ib[r] = a.pairing == 0 ? 2 * p + 1 : p + half_rot;
            } else {
                ia[r] = a.rotary_dim + 2 * (p - half_rot);
                ib[r] = ia[r] + 1;
            }
            xa[r] = to_f32<TX>(x[ia[r]]);
            xb[r] = to_f32<TX>(x[ib[r]]);
            ss += xa[r] * xa[r] + xb[r] * xb[r];
        }
    }
    float inv = 1.f;
    if (w) {
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / static_cast<float>(d) + a.eps);
    }

    // where a key goes
    int64_t kbase = 0, vbase = 0;
    int slot = 0;
    bool store_kv = false;
    if (!is_q) {
        const int pos = positions[t];
        const int page = block_table[static_cast<int64_t>(token_entry[t]) * a.bt_width + pos / a.page_size];
        slot = pos % a.page_size;
        store_kv = page >= 0 && page < a.num_pages;
        const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
        kbase = (pg * a.page_size + slot) * d;
        vbase = pg * d * a.page_size + slot;
    }

#pragma unroll
    for (int r = 0; r < MAX_PAIRS_PER_LANE; ++r) {
        const int p = lane + r * PULSE_WAVE;
        if (p < npairs) {
            float va = xa[r], vb = xb[r];
            if (w) {
                va = va * inv * to_f32<TW>(w[ia[r]]);
                vb = vb * inv * to_f32<TW>(w[ib[r]]);
            }
            if (p < half_rot && cos_t) {
                const float c = cos_t[static_cast<int64_t>(t) * half_rot + p];
                const float s = sin_t[static_cast<int64_t>(t) * half_rot + p];
                const float ra = va * c - vb * s;
                const float rb = va * s + vb * c;
                va = ra;
                vb = rb;
            }
            if (is_q) {
                x[ia[r]] = from_f32<TX>(va);
                x[ib[r]] = from_f32<TX>(vb);
            } else if (store_kv) {
                kcache[kbase + ia[r]] = from_f32<TC>(va);
                kcache[kbase + ib[r]] = from_f32<TC>(vb);
            }
        }
    }

    if (!is_q && store_kv) {
        const TX* v = row + static_cast<int64_t>(a.nq + a.nkv + g) * d;
        for (int i = lane; i < d; i += PULSE_WAVE)
            vcache[vbase + static_cast<int64_t>(i) * a.page_size] = from_f32<TC>(to_f32<TX>(v[i]));
    }
}

}  // namespace

extern "C" int pulse_qk_rope_kv(void* qkv, int x_dtype, int64_t row_stride, const void* q_w, const void* k_w,
                                int w_dtype, float eps, const float* cos_t, const float* sin_t, int rotary_dim,
                                int pairing, void* kcache, void* vcache, int c_dtype, const int* positions,
                                const int* token_entry, const int* block_table, int bt_width, int tokens, int nq,
                                int nkv, int d, int page_size, int num_pages, int write_kv, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && nq > 0 && nkv >= 0 && d > 0, "qk_rope_kv: bad sizes");
    PULSE_REQUIRE(d % 2 == 0 && d <= 2 * PULSE_WAVE * MAX_PAIRS_PER_LANE,
                  "qk_rope_kv: head_dim %d must be even and at most %d", d, 2 * PULSE_WAVE * MAX_PAIRS_PER_LANE);
    PULSE_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0,
                  "qk_rope_kv: rotary_dim %d must be even and at most head_dim %d", rotary_dim, d);
    PULSE_REQUIRE(pairing == 0 || pairing == 1, "qk_rope_kv: unknown pairing %d", pairing);
    PULSE_REQUIRE((q_w == nullptr) == (k_w == nullptr), "qk_rope_kv: give both norm weights or neither");
    PULSE_REQUIRE(rotary_dim == 0 || (cos_t && sin_t), "qk_rope_kv: rotation needs the cos/sin tables");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(c_dtype), "qk_rope_kv: bad dtype tag");
    PULSE_REQUIRE(qkv && positions, "qk_rope_kv: null pointer");
    if (write_kv) {
        PULSE_REQUIRE(kcache && vcache && token_entry && block_table, "qk_rope_kv: cache pointers missing");
        PULSE_REQUIRE(page_size > 0 && num_pages > 0 && bt_width > 0 && nkv > 0, "qk_rope_kv: bad cache geometry");
        PULSE_REQUIRE(row_stride >= static_cast<int64_t>(nq + 2 * nkv) * d, "qk_rope_kv: row stride too small");
    } else {
        PULSE_REQUIRE(row_stride >= static_cast<int64_t>(nq) * d, "qk_rope_kv: row stride too small");
    }
    if (tokens == 0) return 0;
    QkRopeArgs a;
    a.nq = nq; a.nkv = nkv; a.d = d; a.row_stride = row_stride; a.eps = eps;
    a.rotary_dim = (cos_t ? rotary_dim : 0); a.pairing = pairing;
    a.page_size = page_size; a.num_pages = num_pages; a.bt_width = bt_width; a.write_kv = write_kv;
    const dim3 grid(tokens, write_kv ? nq + nkv : nq);
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        hipLaunchKernelGGL((qk_rope_kv_kernel<TX, TW, TC>), grid, dim3(64), 0, stream, static_cast<TX*>(qkv),
                           static_cast<const TW*>(q_w), static_cast<const TW*>(k_w), cos_t, sin_t,
                           static_cast<TC*>(kcache), static_cast<TC*>(vcache), positions, token_entry,
                           block_table, a))));
    PULSE_LAUNCH_CHECK("qk_rope_kv");
    return 0;
}
