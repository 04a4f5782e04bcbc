// Choosing the next token from float32 logits, one workgroup per row.
//
// The steps and their order are the reference sampler's
// (reference: demo/qwen3_infer.cpp:230-423):
//   1. presence penalty: subtract it from every token the request has seen;
//   2. banned ids are removed;
//   3. temperature <= 0: the largest logit wins, the lowest index among equals
//      (reference: src/scheduler/continuous_batch_engine.cpp:20-62);
//   4. top-k: keep the k largest;
//   5. weights exp((l - max) / temperature);
//   6. top-p in (0, 1): keep the most likely tokens whose mass first reaches
//      top_p of the total;
//   7. draw: u * (kept mass), walked along the cumulative sum.
// Differences, both of measure zero or none in distribution: the kept sets are
// found as thresholds (tokens equal to the threshold are all kept), and the
// cumulative walk runs in vocabulary order rather than sorted order.  The
// uniform number u comes from the host's per-request counter-based generator,
// so a row's result does not depend on the other rows.
#include "common.h"

#include <math.h>

namespace {

constexpr int SAMPLE_THREADS = 1024;
constexpr int SAMPLE_WAVES = SAMPLE_THREADS / PULSE_WAVE;

__device__ __forceinline__ uint32_t order_key(float f) {
    if (f != f) return 0u;  // NaN sorts lowest
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

struct RowView {
    const float* logits;
    const uint32_t* seen;    // bit per token, or null
    const uint32_t* banned;  // bit per token, or null
    float penalty;
    int vocab;
    __device__ __forceinline__ float at(int i) const {
        if (banned && ((banned[i >> 5] >> (i & 31)) & 1u)) return -INFINITY;
        float x = logits[i];
        if (x != x) return -INFINITY;
        if (seen && ((seen[i >> 5] >> (i & 31)) & 1u)) x -= penalty;
        return x;
    }
};

__device__ float block_sum_f(float v, float* scratch) { return block_sum(v, scratch); }

__device__ int block_sum_i(int v, int* scratch) {
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PULSE_WAVE);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    int total = 0;
    for (int w = 0; w < SAMPLE_WAVES; ++w) total += scratch[w];
    return total;
}

// (value, index) maximum with the lowest index among equal values
__device__ void block_argmax(float& v, int& idx, float* sv, int* si) {
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, PULSE_WAVE);
        const int oi = __shfl_xor(idx, off, PULSE_WAVE);
        if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
    }
    __syncthreads();
    if (lane == 0) { sv[wave] = v; si[wave] = idx; }
    __syncthreads();
    v = sv[0]; idx = si[0];
    for (int w = 1; w < SAMPLE_WAVES; ++w)
        if (sv[w] > v || (sv[w] == v && si[w] < idx)) { v = sv[w]; idx = si[w]; }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int vocab, int64_t row_stride, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
    const float* __restrict__ penalty, const int* __restrict__ seen_row, const uint32_t* __restrict__ seen_masks,
    const uint32_t* __restrict__ banned, int mask_words, int* __restrict__ out) {
    __shared__ float sf[SAMPLE_WAVES];
    __shared__ int si[SAMPLE_WAVES];
    __shared__ float chunk_sum[SAMPLE_THREADS];
    __shared__ int chosen_thread;
    __shared__ float chosen_rest;

    const int r = blockIdx.x;
    RowView row;
    row.logits = logits + r * row_stride;
    row.vocab = vocab;
    row.banned = banned;
    row.penalty = penalty ? penalty[r] : 0.f;
    row.seen = (seen_masks && seen_row && seen_row[r] >= 0 && row.penalty > 0.f)
                   ? seen_masks + static_cast<int64_t>(seen_row[r]) * mask_words : nullptr;

    // largest logit, lowest index among equals
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
        const float x = row.at(i);
        if (x > best) { best = x; best_i = i; }
    }
    block_argmax(best, best_i, sf, si);
    if (best_i == 0x7fffffff) {  // everything banned or NaN
        if (threadIdx.x == 0) out[r] = -1;
        return;
    }
    const float temp = temperature ? temperature[r] : 0.f;
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[r] = best_i;
        return;
    }

    // top-k threshold: the k-th largest key, found bit by bit
    uint32_t keep = 0u;
    const int k = top_k ? top_k[r] : 0;
    if (k > 0 && k < vocab) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = keep | (1u << bit);
            int count = 0;
            for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) count += order_key(row.at(i)) >= cand;
            if (block_sum_i(count, si) >= k) keep = cand;
        }
    }
    const float inv_t = 1.0f / temp;
    // total mass of what top-k keeps
    float mass = 0.f;
    for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
        const float x = row.at(i);
        if (x != -INFINITY && order_key(x) >= keep) mass += expf((x - best) * inv_t);
    }
    float total = block_sum_f(mass, sf);

    const float p = top_p ? top_p[r] : 0.f;
    if (p > 0.f && p < 1.f) {
        const float want = p * total;
        uint32_t thr = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = thr | (1u << bit);
            const uint32_t lim = cand > keep ? cand : keep;
            float part = 0.f;
            for (int i = threadIdx.x; i < vocab; i += SAMPLE_THREADS) {
                const float x = row.at(i);
                if (x != -INFINITY && order_key(x) >= lim) part += expf((x - best) * inv_t);
            }
            if (block_sum_f(part, sf) >= want) thr = cand;
        }
        if (thr > keep) keep = thr;
    }

    // cumulative walk in vocabulary order over contiguous chunks
    const int chunk = (vocab + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int begin = threadIdx.x * chunk;
    const int end = min(vocab, begin + chunk);
    float mine = 0.f;
    for (int i = begin; i < end; ++i) {
        const float x = row.at(i);
        if (x != -INFINITY && order_key(x) >= keep) mine += expf((x - best) * inv_t);
    }
    chunk_sum[threadIdx.x] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        float kept = 0.f;
        for (int i = 0; i < SAMPLE_THREADS; ++i) kept += chunk_sum[i];
        const float target = uniform[r] * kept;
        float run = 0.f;
        int who = -1;
        for (int i = 0; i < SAMPLE_THREADS; ++i) {
            if (chunk_sum[i] > 0.f && target < run + chunk_sum[i]) { who = i; break; }
            run += chunk_sum[i];
        }
        chosen_thread = who;
        chosen_rest = target - run;
        if (who < 0) out[r] = best_i;  // rounding left the target beyond the last chunk
    }
    __syncthreads();
    if (static_cast<int>(threadIdx.x) == chosen_thread) {
        float run = 0.f;
        int pick = -1, last = -1;
        for (int i = begin; i < end; ++i) {
            const float x = row.at(i);
            if (x != -INFINITY && order_key(x) >= keep) {
                run += expf((x - best) * inv_t);
                last = i;
                if (chosen_rest < run) { pick = i; break; }
            }
        }
        out[r] = pick >= 0 ? pick : (last >= 0 ? last : best_i);
    }
}

__global__ void mark_seen_kernel(uint32_t* __restrict__ masks, int mask_words, const int* __restrict__ rows,
                                 const int* __restrict__ tokens, int n, int vocab) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int tok = tokens[i];
    if (tok < 0 || tok >= vocab || rows[i] < 0) return;
    atomicOr(masks + static_cast<int64_t>(rows[i]) * mask_words + (tok >> 5), 1u << (tok & 31));
}

// Greedy choice in two stages so that a few rows of a large vocabulary use the whole chip:
// each workgroup scans one chunk of a row, then one workgroup per row merges the chunk winners.
constexpr int ARGMAX_THREADS = 256;

__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_chunks_kernel(const float* __restrict__ logits, int vocab,
                                                                       int64_t row_stride, int chunk,
                                                                       float* __restrict__ part_val,
                                                                       int* __restrict__ part_idx) {
    __shared__ float sv[ARGMAX_THREADS / PULSE_WAVE];
    __shared__ int si[ARGMAX_THREADS / PULSE_WAVE];
    const int r = blockIdx.y;
    const int begin = blockIdx.x * chunk;
    const int end = min(vocab, begin + chunk);
    const float* row = logits + r * row_stride;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += ARGMAX_THREADS) {
        const float x = row[i];
        if (x > best) { best = x; best_i = i; }   // NaN never wins; ascending i keeps the lowest index among equals
    }
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, PULSE_WAVE);
        const int oi = __shfl_xor(best_i, off, PULSE_WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (lane == 0) { sv[wave] = best; si[wave] = best_i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < ARGMAX_THREADS / PULSE_WAVE; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < best_i)) { best = sv[w]; best_i = si[w]; }
        part_val[r * gridDim.x + blockIdx.x] = best;
        part_idx[r * gridDim.x + blockIdx.x] = best_i;
    }
}

__global__ __launch_bounds__(PULSE_WAVE) void argmax_merge_kernel(const float* __restrict__ part_val,
                                                                  const int* __restrict__ part_idx, int chunks,
                                                                  int* __restrict__ out) {
    const int r = blockIdx.x;
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int c = threadIdx.x; c < chunks; c += PULSE_WAVE) {
        const float v = part_val[r * chunks + c];
        const int i = part_idx[r * chunks + c];
        if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
    }
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, PULSE_WAVE);
        const int oi = __shfl_xor(best_i, off, PULSE_WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    if (threadIdx.x == 0) out[r] = best_i == 0x7fffffff ? -1 : best_i;
}

}  // namespace

// out[r] = index of the largest logit of row r, the lowest index among equals, -1 if none is a number.
// part_val / part_idx: scratch of rows * pulse_argmax_chunks(vocab) entries each.
extern "C" int pulse_argmax_chunks(int vocab) {
    const int chunk = 2048;
    return (vocab + chunk - 1) / chunk;
}

extern "C" int pulse_argmax(const float* logits, int rows, int vocab, int64_t row_stride, float* part_val,
                            int* part_idx, int* out, hipStream_t stream) {
    PULSE_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax: bad sizes rows=%d V=%d", rows, vocab);
    PULSE_REQUIRE(rows < 65536, "argmax: at most 65535 rows");
    PULSE_REQUIRE(logits && part_val && part_idx && out, "argmax: null pointer");
    if (rows == 0) return 0;
    const int chunks = pulse_argmax_chunks(vocab);
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(chunks, rows), dim3(ARGMAX_THREADS), 0, stream, logits, vocab,
                       row_stride, 2048, part_val, part_idx);
    PULSE_LAUNCH_CHECK("argmax_chunks");
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(PULSE_WAVE), 0, stream, part_val, part_idx, chunks, out);
    PULSE_LAUNCH_CHECK("argmax_merge");
    return 0;
}

// out[r] = chosen token of row r, or -1 when no token is allowed.
// temperature/top_k/top_p/penalty/seen_row/banned may be null (greedy, off, off, none, none, none).
extern "C" int pulse_sample(const float* logits, int rows, int vocab, int64_t row_stride, const float* temperature,
                            const int* top_k, const float* top_p, const float* uniform, const float* penalty,
                            const int* seen_row, const uint32_t* seen_masks, const uint32_t* banned,
                            int mask_words, int* out, hipStream_t stream) {
    PULSE_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample: bad sizes rows=%d V=%d", rows, vocab);
    PULSE_REQUIRE(logits && out, "sample: null pointer");
    PULSE_REQUIRE(!temperature || uniform, "sample: temperature sampling needs uniform numbers");
    PULSE_REQUIRE((!seen_masks && !banned) || mask_words * 32 >= vocab, "sample: masks cover %d tokens, vocabulary has %d",
                  mask_words * 32, vocab);
    if (rows == 0) return 0;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, vocab, row_stride,
                       temperature, top_k, top_p, uniform, penalty, seen_row, seen_masks, banned, mask_words, out);
    PULSE_LAUNCH_CHECK("sample");
    return 0;
}

// Set the bit of tokens[i] in the mask row rows[i] (the per-request "seen" set of the presence penalty).
extern "C" int pulse_mark_seen(uint32_t* masks, int mask_words, const int* rows, const int* tokens, int n, int vocab,
                               hipStream_t stream) {
    PULSE_REQUIRE(masks && rows && tokens && n >= 0 && mask_words * 32 >= vocab, "mark_seen: bad arguments");
    if (n == 0) return 0;
    hipLaunchKernelGGL(mark_seen_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, masks, mask_words, rows,
                       tokens, n, vocab);
    PULSE_LAUNCH_CHECK("mark_seen");
    return 0;
}
