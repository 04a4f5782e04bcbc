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

    // Every load is issued before anything waits for one: the head's elements, the norm weight, cos and sin, the
    // value head, and the chain position -> block table -> page.  A wavefront lives for little more than one trip
    // to memory then, and the kernel is bound by that time.
    int ia[MAX_PAIRS_PER_LANE], ib[MAX_PAIRS_PER_LANE];
    float xa[MAX_PAIRS_PER_LANE], xb[MAX_PAIRS_PER_LANE], wa[MAX_PAIRS_PER_LANE], wb[MAX_PAIRS_PER_LANE];
    float cs[MAX_PAIRS_PER_LANE], sn[MAX_PAIRS_PER_LANE];
    const int npairs = d / 2;
#pragma unroll
    for (int r = 0; r < MAX_PAIRS_PER_LANE; ++r) {
        const int p = lane + r * PULSE_WAVE;
        ia[r] = ib[r] = 0;
        xa[r] = xb[r] = 0.f;
        wa[r] = wb[r] = cs[r] = 1.f;
        sn[r] = 0.f;
        if (p < npairs) {
            if (p < half_rot) {
                ia[r] = a.pairing == 0 ? 2 * p : p;
                ib[r] = a.pairing == 0 ? 2 * p + 1 : p + half_rot;
                if (cos_t) {
                    cs[r] = cos_t[static_cast<int64_t>(t) * half_rot + p];
                    sn[r] = sin_t[static_cast<int64_t>(t) * half_rot + p];
                }
            } else {
                ia[r] = a.rotary_dim + 2 * (p - half_rot);
                ib[r] = ia[r] + 1;
            }
            xa[r] = to_f32<TX>(x[ia[r]]);
            xb[r] = to_f32<TX>(x[ib[r]]);
            if (w) {
                wa[r] = to_f32<TW>(w[ia[r]]);
                wb[r] = to_f32<TW>(w[ib[r]]);
            }
        }
    }
    float vv[2 * MAX_PAIRS_PER_LANE];
    int pos = 0, entry = 0;
    if (!is_q) {
        pos = positions[t];
        entry = token_entry[t];
        const TX* v = row + static_cast<int64_t>(a.nq + a.nkv + g) * d;
#pragma unroll
        for (int r = 0; r < 2 * MAX_PAIRS_PER_LANE; ++r) {
            const int i = lane + r * PULSE_WAVE;
            vv[r] = i < d ? to_f32<TX>(v[i]) : 0.f;
        }
    }

    // where a key goes
    int64_t kbase = 0, vbase = 0;
    bool store_kv = false;
    if (!is_q) {
        const int page = block_table[static_cast<int64_t>(entry) * a.bt_width + pos / a.page_size];
        const int slot = pos % a.page_size;
        store_kv = page >= 0 && page < a.num_pages;
        const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
        kbase = (pg * a.page_size + slot) * d;
        vbase = pg * d * a.page_size + slot;
    }

    float inv = 1.f;
    if (w) {
        float ss = 0.f;
#pragma unroll
        for (int r = 0; r < MAX_PAIRS_PER_LANE; ++r) ss += xa[r] * xa[r] + xb[r] * xb[r];
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / static_cast<float>(d) + a.eps);
    }

#pragma unroll
    for (int r = 0; r < MAX_PAIRS_PER_LANE; ++r) {
        const int p = lane + r * PULSE_WAVE;
        if (p < npairs) {
            float va = xa[r], vb = xb[r];
            if (w) {
                va = va * inv * wa[r];
                vb = vb * inv * wb[r];
            }
            if (p < half_rot && cos_t) {
                const float ra = va * cs[r] - vb * sn[r];
                const float rb = va * sn[r] + vb * cs[r];
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
#pragma unroll
        for (int r = 0; r < 2 * MAX_PAIRS_PER_LANE; ++r) {
            const int i = lane + r * PULSE_WAVE;
            if (i < d) vcache[vbase + static_cast<int64_t>(i) * a.page_size] = from_f32<TC>(vv[r]);
        }
    }
}


// The bfloat16 path: a head's row of d elements is taken by d / 8 lanes with 16-byte accesses (8 elements a lane),
// so a wavefront takes 64 / LPH heads of one token at once and runs a tenth of the instructions of the kernel
// above, which is what that kernel's time goes to on long prompts.  The sum of squares runs over the LPH lanes of
// a head.  Needs d and rotary_dim to be multiples of 8, LPH = the power of two >= d / 8 (at most 64).
// PAIRING 0: a lane's pairs are (e0, e1) .. (e6, e7) of 8 consecutive elements.  PAIRING 1: a lane takes elements
// 4c .. 4c+3 and their partners half a rotary_dim further on.  Elements beyond rotary_dim are not rotated.
typedef __attribute__((ext_vector_type(4))) float vf4;
typedef __attribute__((ext_vector_type(4))) uint32_t vu4;
typedef __attribute__((ext_vector_type(2))) uint32_t vu2;

template <typename TW>
__device__ __forceinline__ void load8(const TW* p, float (&out)[8]);
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&out)[8]) {
    const vu4 raw = *reinterpret_cast<const vu4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = __uint_as_float(raw[i] << 16);
        out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, float (&out)[8]) {
    const vf4 lo = *reinterpret_cast<const vf4*>(p);
    const vf4 hi = *reinterpret_cast<const vf4*>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[i] = lo[i];
        out[4 + i] = hi[i];
    }
}
template <typename TW>
__device__ __forceinline__ void load4(const TW* p, float* out);
template <>
__device__ __forceinline__ void load4<bf16_t>(const bf16_t* p, float* out) {
    const vu2 raw = *reinterpret_cast<const vu2*>(p);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        out[2 * i] = __uint_as_float(raw[i] << 16);
        out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
}
template <>
__device__ __forceinline__ void load4<float>(const float* p, float* out) {
    const vf4 v = *reinterpret_cast<const vf4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = v[i];
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    return static_cast<uint32_t>(f32_to_bf16(lo)) | (static_cast<uint32_t>(f32_to_bf16(hi)) << 16);
}

template <typename TW, int PAIRING, int LPH>
__global__ __launch_bounds__(64) void qk_rope_kv_vec_kernel(bf16_t* __restrict__ qkv, const TW* __restrict__ q_w,
                                                            const TW* __restrict__ k_w, const float* __restrict__ cos_t,
                                                            const float* __restrict__ sin_t, bf16_t* __restrict__ kcache,
                                                            bf16_t* __restrict__ vcache, const int* __restrict__ positions,
                                                            const int* __restrict__ token_entry,
                                                            const int* __restrict__ block_table, QkRopeArgs a) {
    constexpr int HPW = PULSE_WAVE / LPH;
    const int t = blockIdx.x;
    const int lane = threadIdx.x;
    const int c = lane % LPH;
    const int hh = blockIdx.y * HPW + lane / LPH;
    const int heads = a.write_kv ? a.nq + a.nkv : a.nq;
    const int d = a.d;
    const int half_rot = a.rotary_dim / 2;
    const bool on = hh < heads && c * 8 < d;
    const bool is_q = hh < a.nq;
    const int g = hh - a.nq;
    bf16_t* row = qkv + static_cast<int64_t>(t) * a.row_stride;
    bf16_t* x = row + static_cast<int64_t>(on ? hh : 0) * d;  // q heads, then k heads, one after the other
    const TW* w = is_q ? q_w : k_w;

    // which elements: two groups of four
    const bool rotated = c * 8 < a.rotary_dim;
    int oa = c * 8, ob = c * 8 + 4;  // PAIRING 0, and everything beyond rotary_dim
    if (PAIRING == 1 && rotated) {
        oa = c * 4;
        ob = c * 4 + half_rot;
    }
    if (!on) oa = 0, ob = 4;

    // every load before anything waits for one
    float e[8], wv[8], cs[4], sn[4];
    if (PAIRING == 0) {
        load8<bf16_t>(x + oa, e);
    } else {
        load4<bf16_t>(x + oa, e);
        load4<bf16_t>(x + ob, e + 4);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) wv[i] = 1.f;
    if (w) {
        if (PAIRING == 0) {
            load8<TW>(w + oa, wv);
        } else {
            load4<TW>(w + oa, wv);
            load4<TW>(w + ob, wv + 4);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) cs[i] = 1.f, sn[i] = 0.f;
    if (cos_t && rotated && on) {
        load4<float>(cos_t + static_cast<int64_t>(t) * half_rot + c * 4, cs);
        load4<float>(sin_t + static_cast<int64_t>(t) * half_rot + c * 4, sn);
    }
    const bool is_k = on && !is_q;
    int pos = 0, entry = 0;
    if (is_k) {
        pos = positions[t];
        entry = token_entry[t];
    }
    bool store_kv = false;
    int64_t kbase = 0;
    if (is_k) {
        const int page = block_table[static_cast<int64_t>(entry) * a.bt_width + pos / a.page_size];
        const int slot = pos % a.page_size;
        store_kv = page >= 0 && page < a.num_pages;
        const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
        kbase = (pg * a.page_size + slot) * d;
    }

    if (!on) {
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = 0.f;
    }
    float inv = 1.f;
    if (w) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += e[i] * e[i];
#pragma unroll
        for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, PULSE_WAVE);
        inv = 1.0f / sqrtf(ss / static_cast<float>(d) + a.eps);
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = e[i] * inv * wv[i];
    }
    if (rotated) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int ia = PAIRING == 0 ? 2 * i : i;
            const int ib = PAIRING == 0 ? 2 * i + 1 : i + 4;
            const float va = e[ia], vb = e[ib];
            e[ia] = va * cs[i] - vb * sn[i];
            e[ib] = va * sn[i] + vb * cs[i];
        }
    }
    if (!on) return;
    const vu2 lo = {pack2(e[0], e[1]), pack2(e[2], e[3])};
    const vu2 hi = {pack2(e[4], e[5]), pack2(e[6], e[7])};
    if (is_q) {
        *reinterpret_cast<vu2*>(x + oa) = lo;
        *reinterpret_cast<vu2*>(x + ob) = hi;
    } else if (store_kv) {
        *reinterpret_cast<vu2*>(kcache + kbase + oa) = lo;
        *reinterpret_cast<vu2*>(kcache + kbase + ob) = hi;
    }
}

// The values of the step's tokens into their pages, whose layout has the slots of a page side by side for every
// channel: a workgroup takes 16 consecutive tokens of one kv head, a thread one token (tid % 16) and eight channels
// at a time, so that the 16 lanes of a store write the 16 two-byte slots of one channel, 32 contiguous bytes when
// the tokens fill a page in order (a thread finds its own token's page and slot: any other arrangement is written
// just as correctly, only in smaller pieces).  Written from the kernel above, a token at a time, the same bytes
// took twice as long as everything else that kernel does.
constexpr int VW_TOKENS = 16;
constexpr int VW_THREADS = 256;

__global__ __launch_bounds__(VW_THREADS) void v_page_write_kernel(const bf16_t* __restrict__ qkv, bf16_t* __restrict__ vcache,
                                                                  const int* __restrict__ positions,
                                                                  const int* __restrict__ token_entry,
                                                                  const int* __restrict__ block_table, QkRopeArgs a,
                                                                  int tokens) {
    const int t = blockIdx.x * VW_TOKENS + threadIdx.x % VW_TOKENS;
    const int cg = threadIdx.x / VW_TOKENS;
    const int g = blockIdx.y;
    if (t >= tokens) return;
    const int pos = positions[t];
    const int page = block_table[static_cast<int64_t>(token_entry[t]) * a.bt_width + pos / a.page_size];
    if (page < 0 || page >= a.num_pages) return;
    const int slot = pos % a.page_size;
    const bf16_t* src = qkv + static_cast<int64_t>(t) * a.row_stride + static_cast<int64_t>(a.nq + a.nkv + g) * a.d;
    bf16_t* dst = vcache + (static_cast<int64_t>(page) * a.nkv + g) * a.d * a.page_size + slot;
    for (int c0 = cg * 8; c0 < a.d; c0 += 8 * (VW_THREADS / VW_TOKENS)) {
        const uint4 raw = *reinterpret_cast<const uint4*>(src + c0);
        const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 8; ++i)
            dst[static_cast<int64_t>(c0 + i) * a.page_size] = static_cast<bf16_t>(words[i / 2] >> (16 * (i % 2)));
    }
}

template <typename TW, int PAIRING>
void launch_vec(int lph, dim3 block, hipStream_t stream, int tokens, int heads, bf16_t* qkv, const TW* q_w, const TW* k_w,
                const float* cos_t, const float* sin_t, bf16_t* kcache, bf16_t* vcache, const int* positions,
                const int* token_entry, const int* block_table, const QkRopeArgs& a) {
#define PULSE_VEC(L)                                                                                                    \
    hipLaunchKernelGGL((qk_rope_kv_vec_kernel<TW, PAIRING, L>), dim3(tokens, (heads + 64 / L - 1) / (64 / L)), block, 0,  \
                       stream, qkv, q_w, k_w, cos_t, sin_t, kcache, vcache, positions, token_entry, block_table, a)
    if (lph <= 2) PULSE_VEC(2);
    else if (lph <= 4) PULSE_VEC(4);
    else if (lph <= 8) PULSE_VEC(8);
    else if (lph <= 16) PULSE_VEC(16);
    else if (lph <= 32) PULSE_VEC(32);
    else PULSE_VEC(64);
#undef PULSE_VEC
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
    const int heads = write_kv ? nq + nkv : nq;
    // the 16-byte path: bfloat16 activations and cache, 8-element chunks that the rotation does not cut
    const bool vec = x_dtype == PULSE_BF16 && (!write_kv || c_dtype == PULSE_BF16) && d % 8 == 0 && a.rotary_dim % 8 == 0 && row_stride % 8 == 0 &&
                     (reinterpret_cast<uintptr_t>(qkv) % 16) == 0 && (reinterpret_cast<uintptr_t>(kcache) % 16) == 0 &&
                     (q_w == nullptr || ((reinterpret_cast<uintptr_t>(q_w) % 16) == 0 && (reinterpret_cast<uintptr_t>(k_w) % 16) == 0)) &&
                     (cos_t == nullptr || ((reinterpret_cast<uintptr_t>(cos_t) % 16) == 0 && (reinterpret_cast<uintptr_t>(sin_t) % 16) == 0));
    if (vec) {
        const int lph = d / 8;
        PULSE_DISPATCH_DTYPE(w_dtype, TW,
            if (pairing == 0)
                launch_vec<TW, 0>(lph, dim3(64), stream, tokens, heads, static_cast<bf16_t*>(qkv), static_cast<const TW*>(q_w),
                                  static_cast<const TW*>(k_w), cos_t, sin_t, static_cast<bf16_t*>(kcache),
                                  static_cast<bf16_t*>(vcache), positions, token_entry, block_table, a);
            else
                launch_vec<TW, 1>(lph, dim3(64), stream, tokens, heads, static_cast<bf16_t*>(qkv), static_cast<const TW*>(q_w),
                                  static_cast<const TW*>(k_w), cos_t, sin_t, static_cast<bf16_t*>(kcache),
                                  static_cast<bf16_t*>(vcache), positions, token_entry, block_table, a));
        PULSE_LAUNCH_CHECK("qk_rope_kv");
        if (write_kv) {
            hipLaunchKernelGGL(v_page_write_kernel, dim3((tokens + VW_TOKENS - 1) / VW_TOKENS, nkv), dim3(VW_THREADS), 0, stream,
                               static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(vcache), positions, token_entry,
                               block_table, a, tokens);
            PULSE_LAUNCH_CHECK("v_page_write");
        }
        return 0;
    }
    const dim3 grid(tokens, heads);
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        hipLaunchKernelGGL((qk_rope_kv_kernel<TX, TW, TC>), grid, dim3(64), 0, stream, static_cast<TX*>(qkv),
                           static_cast<const TW*>(q_w), static_cast<const TW*>(k_w), cos_t, sin_t,
                           static_cast<TC*>(kcache), static_cast<TC*>(vcache), positions, token_entry,
                           block_table, a))));
    PULSE_LAUNCH_CHECK("qk_rope_kv");
    return 0;
}
