// Shared helpers for the gfx950 kernels: storage types, wave64 reductions and
// the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Storage type tags used across the C ABI.
enum PulseDType : int { PULSE_F32 = 0, PULSE_BF16 = 1 };

typedef uint16_t bf16_t;  // raw bfloat16 bits

#define PULSE_WAVE 64

// Every entry point returns 0 on success; otherwise a message is left for
// pulse_last_error().  Arguments are checked on the host before any launch.
extern "C" const char* pulse_last_error();
void pulse_set_error(const char* fmt, ...);
int pulse_compute_units();  // of the current device, asked once

#define PULSE_REQUIRE(cond, ...)            \
    do {                                    \
        if (!(cond)) {                      \
            pulse_set_error(__VA_ARGS__);   \
            return 1;                       \
        }                                   \
    } while (0)

#define PULSE_LAUNCH_CHECK(name)                                                  \
    do {                                                                          \
        hipError_t e_ = hipGetLastError();                                        \
        if (e_ != hipSuccess) {                                                   \
            pulse_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return 2;                                                             \
        }                                                                         \
    } while (0)

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// Round to nearest, ties to even; NaN stays NaN.  (The conversion instruction of gfx950, v_cvt_pk_bf16_f32: one
// instruction for two values where the rounding written out in integer arithmetic takes six a value.)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    return __builtin_bit_cast(bf16_t, static_cast<__bf16>(f));
}

// 16 bytes of a tensor that a kernel reads once (weights, the cache): a load marked nontemporal, which the memory
// system streams instead of keeping in its caches.  A plain read of 2 GB runs at 5.9 TB/s with ordinary loads and at
// 6.4 to 6.6 TB/s with these.
typedef __attribute__((ext_vector_type(4))) int pulse_i32x4;
__device__ __forceinline__ pulse_i32x4 stream_load16(const void* p) {
    return __builtin_nontemporal_load(static_cast<const pulse_i32x4*>(p));
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PULSE_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PULSE_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds one float per wave (>= 16).
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x % PULSE_WAVE;
    const int wave = threadIdx.x / PULSE_WAVE;
    const int nwaves = (blockDim.x + PULSE_WAVE - 1) / PULSE_WAVE;
    v = wave_sum(v);
    __syncthreads();  // scratch may still be read from an earlier call
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += scratch[w];  // same order in every thread
    return total;
}

// Dispatch a two-way storage tag to a template argument.
#define PULSE_DISPATCH_DTYPE(tag, T, ...)                 \
    do {                                                  \
        if ((tag) == PULSE_F32) {                         \
            using T = float;                              \
            __VA_ARGS__;                                  \
        } else {                                          \
            using T = bf16_t;                             \
            __VA_ARGS__;                                  \
        }                                                 \
    } while (0)

static inline bool pulse_dtype_ok(int tag) { return tag == PULSE_F32 || tag == PULSE_BF16; }
