// Row-wise kernels around the matrix products: embedding gather, residual add
// fused with RMSNorm (optionally on gathered rows), SwiGLU, and the rotation
// table of the position encoding.  All arithmetic is float32 (the rotation
// angle float64); storage types are template arguments.
#include "common.h"


// ------------------------------------------------------------------ embedding
// out[t, :] = table[ids[t], :] widened to float32 (the residual stream).
// Ids are checked on the host; a bad id here still reads nothing out of range:
// its row becomes NaN, which every later product carries into that token's logits
// (no token is then chosen for it), and *bad_id is raised for a caller that asks.
// (reference: src/ops/kernels/cuda/embedding_kernel.cu:7-28 leaves zeros silently)
template <typename TW>
__global__ void embed_gather_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                                    float* __restrict__ out, int hidden, int vocab, int* bad_id) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* dst = out + static_cast<int64_t>(t) * hidden;
    if (id < 0 || id >= vocab) {
        for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = __builtin_nanf("");
        if (threadIdx.x == 0) *bad_id = 1;
        return;
    }
    const TW* src = table + static_cast<int64_t>(id) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_f32<TW>(src[i]);
}

extern "C" int pulse_embed_gather(const int* ids, const void* table, int table_dtype, float* out,
                                  int tokens, int hidden, int vocab, int* bad_id, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes T=%d H=%d V=%d", tokens, hidden, vocab);
    PULSE_REQUIRE(pulse_dtype_ok(table_dtype), "embed_gather: bad dtype tag %d", table_dtype);
    PULSE_REQUIRE(ids && table && out && bad_id, "embed_gather: null pointer");
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(table_dtype, TW,
        hipLaunchKernelGGL(embed_gather_kernel<TW>, dim3(tokens), dim3(256), 0, stream, ids,
                           static_cast<const TW*>(table), out, hidden, vocab, bad_id));
    PULSE_LAUNCH_CHECK("embed_gather");
    return 0;
}

// --------------------------------------------------- residual add + RMSNorm
// For output row r (input row s = rows ? rows[r] : r):
//   v = h[s] + delta[s]            (delta optional)
//   h[s] = v                       (only when write_back)
//   y[r] = v * (1 / sqrt(mean(v^2) + eps)) * w      one rounding at the end
// (formula: src/ops/kernels/cuda/rmsnorm_kernel.cu:97-157; the reference adds the
// residual in a separate kernel, src/ops/kernels/cuda/add_kernel.cu:73-92)
template <typename TD, typename TW, typename TY>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta, int parts, int64_t part_stride,
                                   const int* __restrict__ rows, const TW* __restrict__ w,
                                   TY* __restrict__ y, int hidden, float eps, int write_back) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int64_t s = rows ? rows[r] : r;
    float* hrow = h + s * hidden;
    const TD* drow = delta ? delta + s * hidden : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = hrow[i];
        if (drow)
            for (int p = 0; p < parts; ++p) v += to_f32<TD>(drow[p * part_stride + i]);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(hidden) + eps);
    TY* yrow = y + static_cast<int64_t>(r) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = hrow[i];
        if (drow)
            for (int p = 0; p < parts; ++p) v += to_f32<TD>(drow[p * part_stride + i]);
        if (write_back) hrow[i] = v;
        yrow[i] = from_f32<TY>(v * inv * to_f32<TW>(w[i]));
    }
}

// The same for rows of up to 256 * 4 * RMS_CHUNKS values with hidden % 4 == 0: one pass, the row held in
// registers, 16-byte accesses.  Few rows (decoding) are bound by latency, and this halves the dependent loads.
constexpr int RMS_CHUNKS = 8;

template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float4 type; };
template <> struct Vec4<bf16_t> { typedef ushort4 type; };

__device__ __forceinline__ float4 widen4(float4 v) { return v; }
__device__ __forceinline__ float4 widen4(ushort4 v) {
    return make_float4(bf16_to_f32(v.x), bf16_to_f32(v.y), bf16_to_f32(v.z), bf16_to_f32(v.w));
}
template <typename T> __device__ __forceinline__ typename Vec4<T>::type narrow4(float4 v);
template <> __device__ __forceinline__ float4 narrow4<float>(float4 v) { return v; }
template <> __device__ __forceinline__ ushort4 narrow4<bf16_t>(float4 v) {
    return make_ushort4(f32_to_bf16(v.x), f32_to_bf16(v.y), f32_to_bf16(v.z), f32_to_bf16(v.w));
}

// THREADS threads a row: 256, or 1024 for few rows and for an update in parts (a row then has enough loads in
// flight to be read at more than the rate of one wavefront's round trips).
// PARTS: the update may come in parts (kept apart so that the kernel for one update needs no more registers than it did).
template <typename TD, typename TW, typename TY, int THREADS, bool PARTS>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                              int parts, int64_t part_stride,
                                                              const int* __restrict__ rows, const TW* __restrict__ w,
                                                              TY* __restrict__ y, int hidden, float eps, int write_back) {
    __shared__ float scratch[16];
    typedef typename Vec4<TD>::type VD;
    typedef typename Vec4<TW>::type VW;
    typedef typename Vec4<TY>::type VY;
    const int r = blockIdx.x;
    const int64_t s = rows ? rows[r] : r;
    const int nvec = hidden / 4;
    float4* hrow = reinterpret_cast<float4*>(h + s * hidden);
    const VD* drow = delta ? reinterpret_cast<const VD*>(delta + s * hidden) : nullptr;
    constexpr int CHUNKS = RMS_CHUNKS * 256 / THREADS;
    float4 v[CHUNKS];
    float ss = 0.f;
    if (!PARTS) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int i = threadIdx.x + c * THREADS;
            if (i < nvec) {
                v[c] = hrow[i];
                if (drow) {
                    const float4 d = widen4(drow[i]);
                    v[c].x += d.x; v[c].y += d.y; v[c].z += d.z; v[c].w += d.w;
                }
                ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
            }
        }
    } else {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int i = threadIdx.x + c * THREADS;
            if (i < nvec) v[c] = hrow[i];
        }
        // The parts of an update (shares of a product's inner dimension) are added in their order; the loads of
        // several parts are asked for before the first is added, since few rows are bound by the trips to memory.
#pragma unroll 8
        for (int p = 0; p < parts; ++p) {
            float4 d[CHUNKS];
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const int i = threadIdx.x + c * THREADS;
                if (i < nvec) d[c] = widen4(drow[p * (part_stride / 4) + i]);
            }
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const int i = threadIdx.x + c * THREADS;
                if (i < nvec) { v[c].x += d[c].x; v[c].y += d[c].y; v[c].z += d[c].z; v[c].w += d[c].w; }
            }
        }
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int i = threadIdx.x + c * THREADS;
            if (i < nvec) ss += v[c].x * v[c].x + v[c].y * v[c].y + v[c].z * v[c].z + v[c].w * v[c].w;
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(hidden) + eps);
    VY* yrow = reinterpret_cast<VY*>(y + static_cast<int64_t>(r) * hidden);
    const VW* wv = reinterpret_cast<const VW*>(w);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int i = threadIdx.x + c * THREADS;
        if (i < nvec) {
            if (write_back) hrow[i] = v[c];
            const float4 ww = widen4(wv[i]);
            yrow[i] = narrow4<TY>(make_float4(v[c].x * inv * ww.x, v[c].y * inv * ww.y, v[c].z * inv * ww.z,
                                              v[c].w * inv * ww.w));
        }
    }
}

// delta may come in `parts` (>= 1) matrices of the shape of h, `part_stride` elements apart: h + their sum, added in
// order, is what is normalised (the shares of a product whose inner dimension was split).
extern "C" int pulse_add_rmsnorm(float* h, const void* delta, int delta_dtype, int parts, int64_t part_stride,
                                 const int* rows, const void* w, int w_dtype, void* y, int y_dtype, int out_rows,
                                 int hidden, float eps, int write_back, hipStream_t stream) {
    PULSE_REQUIRE(parts >= 1 && (parts == 1 || (delta && part_stride % 4 == 0)), "add_rmsnorm: bad parts of the update");
    PULSE_REQUIRE(out_rows >= 0 && hidden > 0, "add_rmsnorm: bad sizes rows=%d H=%d", out_rows, hidden);
    PULSE_REQUIRE(pulse_dtype_ok(delta_dtype) && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(y_dtype),
                  "add_rmsnorm: bad dtype tag");
    PULSE_REQUIRE(h && w && y, "add_rmsnorm: null pointer");
    PULSE_REQUIRE(!(rows && write_back), "add_rmsnorm: write_back with gathered rows is not supported");
    if (out_rows == 0) return 0;
    const bool aligned = (reinterpret_cast<uintptr_t>(h) % 16 == 0) && (reinterpret_cast<uintptr_t>(y) % 16 == 0) &&
                         (reinterpret_cast<uintptr_t>(w) % 16 == 0) && (reinterpret_cast<uintptr_t>(delta) % 16 == 0);
    if (hidden % 4 == 0 && hidden <= 256 * 4 * RMS_CHUNKS && aligned) {
        PULSE_DISPATCH_DTYPE(delta_dtype, TD, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(y_dtype, TY,
            if (parts > 1)
                hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TW, TY, 1024, true>), dim3(out_rows), dim3(1024), 0, stream, h,
                                   static_cast<const TD*>(delta), parts, part_stride, rows, static_cast<const TW*>(w),
                                   static_cast<TY*>(y), hidden, eps, write_back);
            else if (out_rows <= 256 && hidden >= 2048)   // few rows: bound by round trips, not by bandwidth
                hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TW, TY, 1024, false>), dim3(out_rows), dim3(1024), 0, stream, h,
                                   static_cast<const TD*>(delta), parts, part_stride, rows, static_cast<const TW*>(w),
                                   static_cast<TY*>(y), hidden, eps, write_back);
            else
                hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TW, TY, 256, false>), dim3(out_rows), dim3(256), 0, stream, h,
                                   static_cast<const TD*>(delta), parts, part_stride, rows, static_cast<const TW*>(w),
                                   static_cast<TY*>(y), hidden, eps, write_back))));
    } else {
        PULSE_DISPATCH_DTYPE(delta_dtype, TD, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(y_dtype, TY,
            hipLaunchKernelGGL((add_rmsnorm_kernel<TD, TW, TY>), dim3(out_rows), dim3(256), 0, stream, h,
                               static_cast<const TD*>(delta), parts, part_stride, rows, static_cast<const TW*>(w),
                               static_cast<TY*>(y), hidden, eps, write_back))));
    }
    PULSE_LAUNCH_CHECK("add_rmsnorm");
    return 0;
}

// -------------------------------------------------------------- residual add
// h += delta (used where no norm follows).
template <typename TD>
__global__ void residual_add_kernel(float* __restrict__ h, const TD* __restrict__ delta, int parts, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = h[i];
    for (int p = 0; p < parts; ++p) v += to_f32<TD>(delta[p * n + i]);
    h[i] = v;
}

// delta holds `parts` (>= 1) arrays of n values one after the other; they are added in order.
extern "C" int pulse_residual_add(float* h, const void* delta, int delta_dtype, int parts, int64_t n, hipStream_t stream) {
    PULSE_REQUIRE(n >= 0 && parts >= 1 && pulse_dtype_ok(delta_dtype) && h && delta, "residual_add: bad arguments");
    if (n == 0) return 0;
    const int64_t blocks = (n + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "residual_add: too many elements (%lld)", static_cast<long long>(n));
    PULSE_DISPATCH_DTYPE(delta_dtype, TD,
        hipLaunchKernelGGL(residual_add_kernel<TD>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, h,
                           static_cast<const TD*>(delta), parts, n));
    PULSE_LAUNCH_CHECK("residual_add");
    return 0;
}

// --------------------------------------------------------------------- SwiGLU
// gu is [T, 2*I].  slab == 0: gate in columns [0, I), up in [I, 2I).  slab > 0: gate and up alternate in
// slabs of `slab` columns (gate slab, up slab, ...), the layout of a slab-interleaved weight.
// out[t, i] = silu(g) * u, silu(x) = x / (1 + exp(-x)), product in float32, one rounding.
// (reference: src/ops/kernels/cuda/silu_kernel.cu:82-97 then mul_kernel.cu:39-46, two roundings)
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, int slab, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t t = idx / inter;
    const int i = static_cast<int>(idx - t * inter);
    const T* row = gu + t * 2 * inter;
    const int gi = slab > 0 ? (i / slab) * 2 * slab + i % slab : i;
    const int ui = slab > 0 ? gi + slab : inter + i;
    const float g = to_f32<T>(row[gi]);
    const float u = to_f32<T>(row[ui]);
    const float s = g / (1.0f + expf(-g));
    out[idx] = from_f32<T>(s * u);
}

// Eight outputs a thread with 16-byte accesses, for bfloat16 rows whose sizes allow it.
__global__ void swiglu_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ out, int inter, int slab,
                                     int64_t total8) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total8) return;
    const int per_row = inter / 8;
    const int64_t t = idx / per_row;
    const int i = static_cast<int>(idx - t * per_row) * 8;
    const bf16_t* row = gu + t * 2 * inter;
    const int gi = slab > 0 ? (i / slab) * 2 * slab + i % slab : i;
    const int ui = slab > 0 ? gi + slab : inter + i;
    const uint4 g4 = *reinterpret_cast<const uint4*>(row + gi);
    const uint4 u4 = *reinterpret_cast<const uint4*>(row + ui);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w};
    const uint32_t uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float g0 = __uint_as_float(gw[j] << 16), g1 = __uint_as_float(gw[j] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[j] << 16), u1 = __uint_as_float(uw[j] & 0xffff0000u);
        const float z0 = g0 / (1.0f + expf(-g0)) * u0;
        const float z1 = g1 / (1.0f + expf(-g1)) * u1;
        ow[j] = static_cast<uint32_t>(f32_to_bf16(z0)) | (static_cast<uint32_t>(f32_to_bf16(z1)) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * inter + i) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int pulse_swiglu(const void* gu, void* out, int dtype, int tokens, int inter, int slab, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && inter > 0 && pulse_dtype_ok(dtype) && gu && out, "swiglu: bad arguments");
    PULSE_REQUIRE(slab >= 0 && (slab == 0 || inter % slab == 0), "swiglu: %d columns do not divide into slabs of %d", inter, slab);
    const int64_t total = static_cast<int64_t>(tokens) * inter;
    if (total == 0) return 0;
    const bool wide = dtype == PULSE_BF16 && inter % 8 == 0 && (slab == 0 || slab % 8 == 0) &&
                      reinterpret_cast<uintptr_t>(gu) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (wide) {
        const int64_t total8 = total / 8;
        const int64_t blocks = (total8 + 255) / 256;
        PULSE_REQUIRE(blocks < (1ll << 31), "swiglu: too many elements");
        hipLaunchKernelGGL(swiglu_bf16x8_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const bf16_t*>(gu), static_cast<bf16_t*>(out), inter, slab, total8);
        PULSE_LAUNCH_CHECK("swiglu");
        return 0;
    }
    const int64_t blocks = (total + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "swiglu: too many elements");
    PULSE_DISPATCH_DTYPE(dtype, T,
        hipLaunchKernelGGL(swiglu_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const T*>(gu), static_cast<T*>(out), inter, slab, total));
    PULSE_LAUNCH_CHECK("swiglu");
    return 0;
}

// ------------------------------------------------------------- rotation table
// cos_out/sin_out [T, half]: angle = position * inv_freq[i], the product and the
// functions in float64, then rounded to float32 once.  inv_freq[i] = theta^(-2i/rotary_dim)
// comes from the host in float64.
// (reference angle: src/ops/kernels/cuda/rope_kernel.cu:119-123, float32 throughout)
__global__ void rope_table_kernel(const int* __restrict__ positions, const double* __restrict__ inv_freq,
                                  float* __restrict__ cos_out, float* __restrict__ sin_out, int half, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t t = idx / half;
    const int i = static_cast<int>(idx - t * half);
    const double angle = static_cast<double>(positions[t]) * inv_freq[i];
    double s, c;
    sincos(angle, &s, &c);
    cos_out[idx] = static_cast<float>(c);
    sin_out[idx] = static_cast<float>(s);
}

extern "C" int pulse_rope_table(const int* positions, const double* inv_freq, float* cos_out, float* sin_out,
                                int tokens, int half, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && half > 0 && positions && inv_freq && cos_out && sin_out, "rope_table: bad arguments");
    const int64_t total = static_cast<int64_t>(tokens) * half;
    if (total == 0) return 0;
    const int64_t blocks = (total + 255) / 256;
    hipLaunchKernelGGL(rope_table_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, positions,
                       inv_freq, cos_out, sin_out, half, total);
    PULSE_LAUNCH_CHECK("rope_table");
    return 0;
}

// ------------------------------------------------------------- row gather
// out[r, :] = in[rows[r], :] for float32 rows (used to pick the wanted rows of the residual).
__global__ void gather_rows_kernel(const float* __restrict__ in, const int* __restrict__ rows,
                                   float* __restrict__ out, int hidden) {
    const int r = blockIdx.x;
    const float* src = in + static_cast<int64_t>(rows[r]) * hidden;
    float* dst = out + static_cast<int64_t>(r) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = src[i];
}

extern "C" int pulse_gather_rows(const float* in, const int* rows, float* out, int out_rows, int hidden,
                                 hipStream_t stream) {
    PULSE_REQUIRE(out_rows >= 0 && hidden > 0 && in && rows && out, "gather_rows: bad arguments");
    if (out_rows == 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(out_rows), dim3(256), 0, stream, in, rows, out, hidden);
    PULSE_LAUNCH_CHECK("gather_rows");
    return 0;
}
