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
// With top-k (or top-p alone on a peaked row) the row is read three times: the maximum, a histogram of the values
// that locates the k-th largest, and the collection of what lies at or above its bin; the rest happens on that
// short list in LDS.  Rows that do not fit (many equal values, a flat row under top-p alone) take passes over the
// whole vocabulary for every bit of a threshold, with the same result.
// Differences, both of measure zero or none in distribution: the kept sets are
// found as thresholds (tokens equal to the threshold are all kept), and the
// cumulative walk runs in vocabulary order rather than sorted order.  The
// uniform number u comes from the host's per-request counter-based generator,
// so a row's result does not depend on the other rows.
#include "common.h"
#include "no_alloc.h"

#include <math.h>

#include <mutex>

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
    // (without a branch on what was loaded: the loads of several entries can then be in flight together)
    __device__ __forceinline__ float at(int i) const {
        const float x = logits[i];
        const bool out = banned ? ((banned[i >> 5] >> (i & 31)) & 1u) != 0u : false;
        const bool was = seen ? ((seen[i >> 5] >> (i & 31)) & 1u) != 0u : false;
        return (out || x != x) ? -INFINITY : (was ? x - penalty : x);
    }
};

// f(i, value) for i = first, first + step, .. below end, in that order; the values of eight entries are asked for
// before the first is used (a workgroup alone on its row otherwise waits out a trip to memory for every entry).
template <typename F>
__device__ __forceinline__ void sweep(const RowView& row, int first, int end, int step, F f) {
    constexpr int AHEAD = 8;
    int i = first;
    for (; i + (AHEAD - 1) * step < end; i += AHEAD * step) {
        float x[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) x[u] = row.at(i + u * step);
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) f(i + u * step, x[u]);
    }
    for (; i < end; i += step) f(i, row.at(i));
}

__device__ float block_sum_f(float v, float* scratch) { return block_sum(v, scratch); }

__device__ float block_max_f(float v, float* scratch) {
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PULSE_WAVE));
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float m = scratch[0];
    for (int w = 1; w < SAMPLE_WAVES; ++w) m = fmaxf(m, scratch[w]);
    return m;
}

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

// ---- the walk along the cumulative sum, a wavefront over 64 consecutive entries at a time ---------------------
// `weight(i)` is the weight of entry i of [begin, end) (0 for what is not kept), entries in vocabulary order.  The
// wavefront finds the first entry at which the running sum exceeds `rest` and returns its number, or -1 if the sum
// never gets there (rounding); `last` is the last entry with a weight.  Every lane returns the same.
template <typename Weight>
__device__ int wave_walk(int begin, int end, float rest, Weight weight, int& last) {
    const int lane = threadIdx.x % PULSE_WAVE;
    constexpr int AHEAD = 8;   // steps of 64 entries whose weights are asked for together (a step's trip to memory
                               // would otherwise be waited for before the next one starts)
    float run = 0.f;
    last = -1;
    for (int first = begin; first < end; first += AHEAD * PULSE_WAVE) {
        float ws[AHEAD];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int i = first + u * PULSE_WAVE + lane;
            ws[u] = i < end ? weight(i) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int base = first + u * PULSE_WAVE;
            const float w = ws[u];
            const unsigned long long has = __ballot(w > 0.f);
            if (has == 0ull) continue;
            last = base + (63 - __builtin_clzll(has));
            // inclusive prefix over the lanes, in lane order
            float pre = w;
#pragma unroll
            for (int off = 1; off < PULSE_WAVE; off <<= 1) {
                const float up = __shfl_up(pre, off, PULSE_WAVE);
                if (lane >= off) pre += up;
            }
            const unsigned long long hit = __ballot(w > 0.f && rest < run + pre);
            if (hit != 0ull) return base + __builtin_ctzll(hit);
            run += __shfl(pre, PULSE_WAVE - 1, PULSE_WAVE);
        }
    }
    return -1;
}

constexpr int HIST_BINS = 2048;                         // bins of the value histogram that locates the k-th largest
constexpr int WAVE_CAP = 128;                           // candidates a wavefront may collect
constexpr int LIST_CAP = SAMPLE_WAVES * WAVE_CAP;       // candidates of a row
constexpr int LIST_PER_LANE = LIST_CAP / PULSE_WAVE;

// The end of the choice on a short list in LDS, by one wavefront: `n` candidates in vocabulary order (`list_i`, their
// values `list_x`, which are overwritten), among them every token that top-k keeps.  The k-th largest value by a
// search bit by bit, then top-p on what that kept (relative to its mass; without top-k relative to `whole`, the mass
// of the whole row, and only if the list holds that much: else false and nothing is chosen), then the walk along the
// cumulative sum.  Every lane returns the same.  PER: entries a lane takes (n <= PER * 64).
template <int PER>
__device__ bool finish_on_list(const int* list_i, float* list_x, int n, bool by_k, int k, bool use_p, float p, float whole,
                               float best, float inv_t, float u, int best_i, int& token) {
    const int lane = threadIdx.x % PULSE_WAVE;
    auto lane_sum_i = [&](int v) {
#pragma unroll
        for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PULSE_WAVE);
        return v;
    };
    auto lane_sum_f = [&](float v) {
#pragma unroll
        for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PULSE_WAVE);
        return v;
    };
    uint32_t keys[PER];
    float wts[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = lane + j * PULSE_WAVE;
        keys[j] = e < n ? order_key(list_x[e]) : 0u;
        wts[j] = e < n ? expf((list_x[e] - best) * inv_t) : 0.f;
    }
    // the k-th largest key, bit by bit
    uint32_t keep = 0u;
    if (by_k) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = keep | (1u << bit);
            int c = 0;
#pragma unroll
            for (int j = 0; j < PER; ++j) c += (lane + j * PULSE_WAVE < n && keys[j] >= cand) ? 1 : 0;
            if (lane_sum_i(c) >= k) keep = cand;
        }
    }
    if (use_p) {
        float mass = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j) mass += keys[j] >= keep ? wts[j] : 0.f;
        mass = lane_sum_f(mass);
        const float want = p * (by_k ? mass : whole);
        if (!by_k && !(mass >= want)) return false;   // without top-k the list must hold all of the top_p set
        uint32_t thr = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = thr | (1u << bit);
            const uint32_t lim = cand > keep ? cand : keep;
            float part_mass = 0.f;
#pragma unroll
            for (int j = 0; j < PER; ++j) part_mass += keys[j] >= lim ? wts[j] : 0.f;
            if (lane_sum_f(part_mass) >= want) thr = cand;
        }
        if (thr > keep) keep = thr;
    }
    // what is kept, as weights in the list's place of x, then the walk
    float kept = 0.f;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = lane + j * PULSE_WAVE;
        const float w = (e < n && keys[j] >= keep) ? wts[j] : 0.f;
        if (e < n) list_x[e] = w;
        kept += w;
    }
    kept = lane_sum_f(kept);
    int last;
    const int e = wave_walk(0, n, u * kept, [&](int q) { return list_x[q]; }, last);
    token = e >= 0 ? list_i[e] : (last >= 0 ? list_i[last] : best_i);
    return true;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int vocab, int64_t row_stride, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
    const float* __restrict__ penalty, const int* __restrict__ seen_row, const uint32_t* __restrict__ seen_masks,
    const uint32_t* __restrict__ banned, int mask_words, int* __restrict__ out, const int* __restrict__ done) {
    __shared__ float sf[SAMPLE_WAVES];
    __shared__ int si[SAMPLE_WAVES];
    __shared__ int hist[HIST_BINS];
    if (done && done[blockIdx.x]) return;   // the kernels that work in chunks have chosen this row's token already
    __shared__ int wave_bins[SAMPLE_WAVES];
    __shared__ int region_i[SAMPLE_WAVES][WAVE_CAP];
    __shared__ float region_x[SAMPLE_WAVES][WAVE_CAP];
    __shared__ int region_n[SAMPLE_WAVES];
    __shared__ int list_i[LIST_CAP];
    __shared__ float list_x[LIST_CAP];
    __shared__ float part_sum[SAMPLE_WAVES];
    __shared__ int list_done;

    const int r = blockIdx.x;
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    RowView row;
    row.logits = logits + r * row_stride;
    row.vocab = vocab;
    row.banned = banned;
    row.penalty = penalty ? penalty[r] : 0.f;
    row.seen = (seen_masks && seen_row && seen_row[r] >= 0 && row.penalty > 0.f)
                   ? seen_masks + static_cast<int64_t>(seen_row[r]) * mask_words : nullptr;

    // largest logit, lowest index among equals; the smallest number too (the histogram's range)
    float best = -INFINITY, lowest = INFINITY;
    int best_i = 0x7fffffff;
    sweep(row, threadIdx.x, vocab, SAMPLE_THREADS, [&](int i, float x) {
        if (x > best) { best = x; best_i = i; }
        if (x != -INFINITY) lowest = fminf(lowest, x);
    });
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
    const float inv_t = 1.0f / temp;
    const int k = top_k ? top_k[r] : 0;
    const float p = top_p ? top_p[r] : 0.f;
    const bool use_p = p > 0.f && p < 1.f;
    // each wavefront owns a contiguous part of the vocabulary, walked 64 entries at a time
    const int part = ((vocab + SAMPLE_WAVES - 1) / SAMPLE_WAVES + PULSE_WAVE - 1) / PULSE_WAVE * PULSE_WAVE;
    const int part_begin = min(vocab, wave * part), part_end = min(vocab, wave * part + part);

    // ---- with top-k: locate the k-th largest with a histogram over [lowest, best], collect what lies at or above
    // its bin (in vocabulary order), and finish on that short list in LDS.  Falls through to the passes over the
    // whole vocabulary when the list would not fit (many equal values) or the range is empty.
    // Top-p alone takes the same way with the LIST_TRY largest values, if their mass reaches top_p of the whole.
    constexpr int LIST_TRY = 1024;
    const bool by_k = k > 0 && k < vocab;
    const int k_list = by_k ? k : min(vocab - 1, LIST_TRY);
    if (by_k || (use_p && k_list > 0)) {
        float whole = 0.f;   // without top-k: the mass of the whole vocabulary, which top_p refers to
        if (!by_k) {
            float mass = 0.f;
            sweep(row, threadIdx.x, vocab, SAMPLE_THREADS, [&](int, float x) {
                if (x != -INFINITY) mass += expf((x - best) * inv_t);
            });
            whole = block_sum_f(mass, sf);
        }
        lowest = -block_max_f(-lowest, sf);
        const float scale = static_cast<float>(HIST_BINS) / (best - lowest);
        const bool ranged = best > lowest && scale < INFINITY;
        auto bin_of = [&](float x) { return min(HIST_BINS - 1, static_cast<int>((best - x) * scale)); };  // 0: the largest values
        int edge = -1, listed = 0;
        if (ranged) {
            for (int b = threadIdx.x; b < HIST_BINS; b += SAMPLE_THREADS) hist[b] = 0;
            __syncthreads();
            sweep(row, threadIdx.x, vocab, SAMPLE_THREADS, [&](int, float x) {
                if (x != -INFINITY) atomicAdd(&hist[bin_of(x)], 1);
            });
            __syncthreads();
            // the bin in which the count from the top reaches k: first by wavefronts' shares of the bins, then by bins
            constexpr int SHARE = HIST_BINS / SAMPLE_WAVES;
            int mine = 0;
            for (int b = wave * SHARE + lane; b < (wave + 1) * SHARE; b += PULSE_WAVE) mine += hist[b];
#pragma unroll
            for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) mine += __shfl_xor(mine, off, PULSE_WAVE);
            if (lane == 0) wave_bins[wave] = mine;
            __syncthreads();
            int w = 0;
            while (w < SAMPLE_WAVES && listed + wave_bins[w] < k_list) listed += wave_bins[w++];
            if (w < SAMPLE_WAVES) {
                int b = w * SHARE;
                while (listed + hist[b] < k_list) listed += hist[b++];
                listed += hist[b];
                edge = b;
            }
        }
        if (edge >= 0 && listed <= LIST_CAP) {
            int count = 0;
            constexpr int AHEAD = 8;   // steps of 64 entries whose values are asked for together
            for (int base = part_begin; base < part_end; base += AHEAD * PULSE_WAVE) {
                float xs[AHEAD];
#pragma unroll
                for (int u = 0; u < AHEAD; ++u) {
                    const int i = base + u * PULSE_WAVE + lane;
                    xs[u] = i < part_end ? row.at(i) : -INFINITY;
                }
#pragma unroll
                for (int u = 0; u < AHEAD; ++u) {
                    const int i = base + u * PULSE_WAVE + lane;
                    const float x = xs[u];
                    const bool in = x != -INFINITY && bin_of(x) <= edge;
                    const unsigned long long mask = __ballot(in);
                    const int at = count + __builtin_popcountll(mask & ((1ull << lane) - 1ull));
                    if (in && at < WAVE_CAP) { region_i[wave][at] = i; region_x[wave][at] = x; }
                    count += __builtin_popcountll(mask);
                }
            }
            if (lane == 0) region_n[wave] = count;
            __syncthreads();
            bool fits = true;
            for (int w = 0; w < SAMPLE_WAVES; ++w) fits = fits && region_n[w] <= WAVE_CAP;
            if (fits) {
                // one list, in vocabulary order
                int n = 0;
                for (int w = 0; w < SAMPLE_WAVES; ++w) {
                    for (int e = threadIdx.x; e < region_n[w]; e += SAMPLE_THREADS) {
                        list_i[n + e] = region_i[w][e];
                        list_x[n + e] = region_x[w][e];
                    }
                    n += region_n[w];
                }
                __syncthreads();
                // the first wavefront finishes alone (lane l holds entries l, l + 64, ..); the others wait for its word
                if (wave == 0) {
                    int token;
                    const bool enough = finish_on_list<LIST_PER_LANE>(list_i, list_x, n, by_k, k, use_p, p, whole, best, inv_t, uniform[r],
                                                       best_i, token);
                    if (lane == 0) {
                        if (enough) out[r] = token;   // else (only without top-k) the list is too short: the passes
                        list_done = enough ? 1 : 0;   // over the whole vocabulary
                    }
                }
                __syncthreads();
                if (list_done) return;
            }
        }
    }

    // ---- passes over the whole vocabulary
    // top-k threshold: the k-th largest key, found bit by bit
    uint32_t keep = 0u;
    if (k > 0 && k < vocab) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = keep | (1u << bit);
            int count = 0;
            sweep(row, threadIdx.x, vocab, SAMPLE_THREADS, [&](int, float x) { count += order_key(x) >= cand; });
            if (block_sum_i(count, si) >= k) keep = cand;
        }
    }
    auto weight_of = [&](float x) { return (x != -INFINITY && order_key(x) >= keep) ? expf((x - best) * inv_t) : 0.f; };
    auto weight = [&](int i) { return weight_of(row.at(i)); };
    if (use_p) {
        float mass = 0.f;
        sweep(row, threadIdx.x, vocab, SAMPLE_THREADS, [&](int, float x) { mass += weight_of(x); });
        const float want = p * block_sum_f(mass, sf);
        // The largest threshold whose kept mass still reaches `want`, four bits of it a pass over the row: the masses
        // above the fifteen candidates of a digit are summed side by side (each in the order in which a pass for it
        // alone would sum it, so the choice is that of a search bit by bit, in an eighth of the passes).
        uint32_t thr = 0u;
        for (int shift = 28; shift >= 0; shift -= 4) {
            float above[15];
#pragma unroll
            for (int j = 0; j < 15; ++j) above[j] = 0.f;
            sweep(row, threadIdx.x, vocab, SAMPLE_THREADS, [&](int, float x) {
                if (x == -INFINITY) return;
                const uint32_t key = order_key(x);
                if (key < keep || key < (thr | (1u << shift))) return;
                const float w = expf((x - best) * inv_t);
#pragma unroll
                for (int j = 0; j < 15; ++j)
                    if (key >= (thr | (static_cast<uint32_t>(j + 1) << shift))) above[j] += w;
            });
            uint32_t digit = 0u;
#pragma unroll
            for (int j = 0; j < 15; ++j)
                if (block_sum_f(above[j], sf) >= want) digit = static_cast<uint32_t>(j + 1);
            thr |= digit << shift;
        }
        if (thr > keep) keep = thr;
    }
    // the kept mass of every wavefront's part, then the part in which the draw falls is walked by its wavefront
    float mine = 0.f;
    sweep(row, part_begin + lane, part_end, PULSE_WAVE, [&](int, float x) { mine += weight_of(x); });
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) mine += __shfl_xor(mine, off, PULSE_WAVE);
    if (lane == 0) part_sum[wave] = mine;
    __syncthreads();
    float kept = 0.f;
    for (int w = 0; w < SAMPLE_WAVES; ++w) kept += part_sum[w];
    const float target = uniform[r] * kept;
    float run = 0.f;
    int who = -1, last_part = -1;
    for (int w = 0; w < SAMPLE_WAVES; ++w) {
        if (part_sum[w] > 0.f) {
            last_part = w;
            if (who < 0 && target < run + part_sum[w]) who = w;
        }
        if (who < 0) run += part_sum[w];
    }
    if (who < 0) {  // rounding left the target beyond the last part: its last kept entry
        who = last_part;
        run = INFINITY;
    }
    if (wave != who) return;
    int last;
    const int e = wave_walk(part_begin, part_end, run == INFINITY ? INFINITY : target - run, weight, last);
    if (lane == 0) out[r] = e >= 0 ? e : (last >= 0 ? last : best_i);
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

// ---- rows in chunks ----------------------------------------------------------------------------------------------
// A workgroup a row reads its row at the rate of one compute unit.  Without top-k and top-p nothing has to be
// known about the row as a whole but its maximum and its mass, so the row is cut into chunks of SIMPLE_CHUNK logits
// with a workgroup each: the chunk's maximum (with its lowest index); then, the row's maximum known, the chunk's
// mass; then one wavefront a row finds the chunk in which u * mass falls (chunk masses summed in chunk order) and
// walks that chunk alone (chunked_choose_kernel).  The steps and their meaning are those of sample_kernel; sums are
// taken in another order.
constexpr int SIMPLE_CHUNK = 2048;
constexpr int SIMPLE_THREADS = 256;

__device__ __forceinline__ RowView simple_row(const float* logits, int r, int64_t row_stride, int vocab,
                                              const float* penalty, const int* seen_row, const uint32_t* seen_masks,
                                              const uint32_t* banned, int mask_words) {
    RowView row;
    row.logits = logits + r * row_stride;
    row.vocab = vocab;
    row.banned = banned;
    row.penalty = penalty ? penalty[r] : 0.f;
    row.seen = (seen_masks && seen_row && seen_row[r] >= 0 && row.penalty > 0.f)
                   ? seen_masks + static_cast<int64_t>(seen_row[r]) * mask_words : nullptr;
    return row;
}

__global__ __launch_bounds__(SIMPLE_THREADS) void simple_max_kernel(
    const float* __restrict__ logits, int vocab, int64_t row_stride, const float* __restrict__ penalty,
    const int* __restrict__ seen_row, const uint32_t* __restrict__ seen_masks, const uint32_t* __restrict__ banned,
    int mask_words, float* __restrict__ part_max, int* __restrict__ part_idx) {
    __shared__ float sv[SIMPLE_THREADS / PULSE_WAVE];
    __shared__ int si[SIMPLE_THREADS / PULSE_WAVE];
    const int r = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const RowView row = simple_row(logits, r, row_stride, vocab, penalty, seen_row, seen_masks, banned, mask_words);
    const int begin = chunk * SIMPLE_CHUNK, end = min(vocab, begin + SIMPLE_CHUNK);
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    sweep(row, begin + static_cast<int>(threadIdx.x), end, SIMPLE_THREADS, [&](int i, float x) {
        if (x > best) { best = x; best_i = i; }   // a thread's indices rise: the first of equals stays
    });
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
        for (int w = 1; w < SIMPLE_THREADS / PULSE_WAVE; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < best_i)) { best = sv[w]; best_i = si[w]; }
        part_max[r * chunks + chunk] = best;
        part_idx[r * chunks + chunk] = best_i;
    }
}

// The row's maximum from the chunks' (every lane gets it).
__device__ __forceinline__ float simple_row_max(const float* part_max, int chunks) {
    float best = -INFINITY;
    for (int c = threadIdx.x % PULSE_WAVE; c < chunks; c += PULSE_WAVE) best = fmaxf(best, part_max[c]);
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) best = fmaxf(best, __shfl_xor(best, off, PULSE_WAVE));
    return best;
}

__global__ __launch_bounds__(SIMPLE_THREADS) void simple_mass_kernel(
    const float* __restrict__ logits, int vocab, int64_t row_stride, const float* __restrict__ temperature,
    const int* __restrict__ top_k,
    const float* __restrict__ penalty, const int* __restrict__ seen_row, const uint32_t* __restrict__ seen_masks,
    const uint32_t* __restrict__ banned, int mask_words, const float* __restrict__ part_max,
    float* __restrict__ part_mass) {
    __shared__ float sf[SIMPLE_THREADS / PULSE_WAVE];
    const int r = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const float temp = temperature ? temperature[r] : 0.f;
    if (!(temp > 0.f)) return;   // the largest logit wins: no mass is asked for
    if (top_k && top_k[r] > 0) return;   // what top-k keeps is weighed on the short list
    const float best = simple_row_max(part_max + r * chunks, chunks);
    if (best == -INFINITY) return;
    const float inv_t = 1.0f / temp;
    const RowView row = simple_row(logits, r, row_stride, vocab, penalty, seen_row, seen_masks, banned, mask_words);
    const int begin = chunk * SIMPLE_CHUNK, end = min(vocab, begin + SIMPLE_CHUNK);
    float mass = 0.f;
    sweep(row, begin + static_cast<int>(threadIdx.x), end, SIMPLE_THREADS, [&](int, float x) {
        if (x != -INFINITY) mass += expf((x - best) * inv_t);
    });
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) mass += __shfl_xor(mass, off, PULSE_WAVE);
    if (lane == 0) sf[wave] = mass;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int w = 0; w < SIMPLE_THREADS / PULSE_WAVE; ++w) total += sf[w];
        part_mass[r * chunks + chunk] = total;
    }
}

// ---- rows with top-k, in chunks -------------------------------------------------------------------------------
// With a small k the candidates can be found chunk by chunk as well.  The k-th largest of the chunks' maxima is a
// lower bound of the k-th largest logit (that many logits, the maxima themselves, reach it), so everything that
// top-k keeps lies at or above it, and little else: a workgroup a chunk collects what it has there, in vocabulary
// order, into its own short segment; a wavefront a row strings the segments together in LDS and finishes on that list
// as sample_kernel does on its own (finish_on_list).  A row that does not fit (k above the number of chunks, a chunk
// with more candidates than its segment holds: many equal values) is left to sample_kernel, which runs behind and
// skips the rows that are done.
constexpr int TOPK_SEGMENT = 32;   // candidates a chunk may leave

// A row with top-p alone takes the same way with what lies at or above one of the lower chunk maxima (seven eighths
// of the chunks have a larger one): some hundreds of the largest logits of a vocabulary of 150,000, which hold the
// top_p share of a distribution as peaked as a language model's; if they do not (or a chunk has more than its segment
// holds), the row is left to sample_kernel too.  The mass of the whole row, which top_p refers to, comes from
// simple_mass_kernel.
__device__ __forceinline__ int top_p_bound_rank(int chunks) { return max(1, chunks - chunks / 8); }

__global__ __launch_bounds__(SIMPLE_THREADS) void topk_collect_kernel(
    const float* __restrict__ logits, int vocab, int64_t row_stride, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ penalty,
    const int* __restrict__ seen_row, const uint32_t* __restrict__ seen_masks, const uint32_t* __restrict__ banned,
    int mask_words, const float* __restrict__ part_max, int* __restrict__ seg_i, float* __restrict__ seg_x,
    int* __restrict__ seg_n) {
    constexpr int WAVES = SIMPLE_THREADS / PULSE_WAVE;
    constexpr int PER = SIMPLE_CHUNK / SIMPLE_THREADS;   // consecutive logits a thread takes
    __shared__ float s_bound;
    __shared__ int s_count[WAVES];
    const int r = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    int k = top_k ? top_k[r] : 0;
    const float p = top_p ? top_p[r] : 0.f;
    if (k <= 0 && p > 0.f && p < 1.f) k = top_p_bound_rank(chunks);   // top-p alone: see top_p_bound_rank
    const float temp = temperature ? temperature[r] : 0.f;
    int* my_n = seg_n + r * chunks + chunk;
    if (!(temp > 0.f) || k <= 0 || k > chunks || chunks > 2 * PULSE_WAVE) {   // greedy rows need no candidates; the others are not for these kernels
        if (threadIdx.x == 0) *my_n = 0;
        return;
    }
    // the chunk's logits are asked for first: they travel while the bound is searched
    const RowView row = simple_row(logits, r, row_stride, vocab, penalty, seen_row, seen_masks, banned, mask_words);
    const int begin = chunk * SIMPLE_CHUNK + static_cast<int>(threadIdx.x) * PER;
    float xs[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int i = begin + j;
        xs[j] = i < vocab ? row.at(i) : -INFINITY;
    }
    // the k-th largest of the chunks' maxima, bit by bit (chunks <= 2 * 64: two a lane)
    if (wave == 0) {
        uint32_t keys[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int c = lane + j * PULSE_WAVE;
            keys[j] = c < chunks ? order_key(part_max[r * chunks + c]) : 0u;
        }
        uint32_t bound = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = bound | (1u << bit);
            int c = (keys[0] >= cand ? 1 : 0) + (keys[1] >= cand ? 1 : 0);
#pragma unroll
            for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) c += __shfl_xor(c, off, PULSE_WAVE);
            if (c >= k) bound = cand;
        }
        // back to the value whose key it is (a maximum of -inf, a chunk with nothing left, has the key of -inf)
        float value = -INFINITY;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int c = lane + j * PULSE_WAVE;
            if (c < chunks && keys[j] == bound) value = part_max[r * chunks + c];
        }
#pragma unroll
        for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) value = fmaxf(value, __shfl_xor(value, off, PULSE_WAVE));
        if (lane == 0) s_bound = value;
    }
    __syncthreads();
    const float bound = s_bound;
    int mine = 0;
#pragma unroll
    for (int j = 0; j < PER; ++j) mine += (xs[j] != -INFINITY && xs[j] >= bound) ? 1 : 0;
    // where this thread's candidates go: an exclusive sum over the threads, in thread order (vocabulary order)
    int pre = mine;
#pragma unroll
    for (int off = 1; off < PULSE_WAVE; off <<= 1) {
        const int up = __shfl_up(pre, off, PULSE_WAVE);
        if (lane >= off) pre += up;
    }
    if (lane == PULSE_WAVE - 1) s_count[wave] = pre;
    __syncthreads();
    int at = pre - mine, total = 0;
    for (int w = 0; w < WAVES; ++w) {
        if (w < wave) at += s_count[w];
        total += s_count[w];
    }
    int* out_i = seg_i + (static_cast<int64_t>(r) * chunks + chunk) * TOPK_SEGMENT;
    float* out_x = seg_x + (static_cast<int64_t>(r) * chunks + chunk) * TOPK_SEGMENT;
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        if (xs[j] != -INFINITY && xs[j] >= bound) {
            if (at < TOPK_SEGMENT) { out_i[at] = begin + j; out_x[at] = xs[j]; }
            ++at;
        }
    }
    if (threadIdx.x == 0) *my_n = total;   // more than TOPK_SEGMENT: the row does not fit
}

// The choice of every row from what the kernels before left, a wavefront a row: the largest logit for greedy rows;
// for rows with top-k the candidates' segments strung together in LDS and finished there; for rows that draw from the
// whole vocabulary the chunk in which u * mass falls (chunk masses in chunk order), walked alone.  done[r] says
// whether the row's token is chosen; the others (rows that did not fit) are sample_kernel's.
__global__ __launch_bounds__(PULSE_WAVE) void chunked_choose_kernel(
    const float* __restrict__ logits, int vocab, int64_t row_stride, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
    const float* __restrict__ penalty, const int* __restrict__ seen_row, const uint32_t* __restrict__ seen_masks,
    const uint32_t* __restrict__ banned, int mask_words, const float* __restrict__ part_max,
    const int* __restrict__ part_idx, const float* __restrict__ part_mass, const int* __restrict__ seg_i,
    const float* __restrict__ seg_x, const int* __restrict__ seg_n, int chunks, int* __restrict__ out,
    int* __restrict__ done) {
    __shared__ int list_i[LIST_CAP];
    __shared__ float list_x[LIST_CAP];
    const int r = blockIdx.x, lane = threadIdx.x;
    part_max += r * chunks;
    part_idx += r * chunks;
    part_mass += r * chunks;
    seg_n += r * chunks;
    // the largest logit, the lowest index among equals
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int c = lane; c < chunks; c += PULSE_WAVE) {
        const float v = part_max[c];
        const int i = part_idx[c];
        if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
    }
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, PULSE_WAVE);
        const int oi = __shfl_xor(best_i, off, PULSE_WAVE);
        if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
    }
    const float temp = temperature ? temperature[r] : 0.f;
    if (best_i == 0x7fffffff || !(temp > 0.f)) {   // everything banned or NaN, or the largest logit wins
        if (lane == 0) { out[r] = best_i == 0x7fffffff ? -1 : best_i; done[r] = 1; }
        return;
    }
    const int k = top_k ? top_k[r] : 0;
    const float p = top_p ? top_p[r] : 0.f;
    const bool use_p = p > 0.f && p < 1.f;
    const float inv_t = 1.0f / temp;
    if (k > 0 || use_p) {
        const bool by_k = k > 0;
        // the segments' places in the list: an exclusive sum over the chunks, in chunk order (two chunks a lane)
        const int n0 = lane < chunks ? seg_n[lane] : 0, n1 = lane + PULSE_WAVE < chunks ? seg_n[lane + PULSE_WAVE] : 0;
        const bool over = n0 > TOPK_SEGMENT || n1 > TOPK_SEGMENT;
        int pre0 = n0, pre1 = n1;
#pragma unroll
        for (int off = 1; off < PULSE_WAVE; off <<= 1) {
            const int u0 = __shfl_up(pre0, off, PULSE_WAVE), u1 = __shfl_up(pre1, off, PULSE_WAVE);
            if (lane >= off) { pre0 += u0; pre1 += u1; }
        }
        const int first = __shfl(pre0, PULSE_WAVE - 1, PULSE_WAVE);      // candidates of chunks 0 .. 63
        const int n = first + __shfl(pre1, PULSE_WAVE - 1, PULSE_WAVE);
        if (k > chunks || chunks > 2 * PULSE_WAVE || __ballot(over) != 0ull || n > LIST_CAP || n < k || n == 0) {
            if (lane == 0) done[r] = 0;   // not a row for these kernels: sample_kernel takes it
            return;
        }
        float whole = 0.f;   // without top-k: the mass of the whole row, chunk masses in chunk order
        if (!by_k) {
            for (int c = lane; c < chunks; c += PULSE_WAVE) whole += part_mass[c];
#pragma unroll
            for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) whole += __shfl_xor(whole, off, PULSE_WAVE);
        }
        const int64_t seg0 = (static_cast<int64_t>(r) * chunks + lane) * TOPK_SEGMENT;
        for (int e = 0; e < n0; ++e) { list_i[pre0 - n0 + e] = seg_i[seg0 + e]; list_x[pre0 - n0 + e] = seg_x[seg0 + e]; }
        const int64_t seg1 = seg0 + static_cast<int64_t>(PULSE_WAVE) * TOPK_SEGMENT;
        for (int e = 0; e < n1; ++e) { list_i[first + pre1 - n1 + e] = seg_i[seg1 + e]; list_x[first + pre1 - n1 + e] = seg_x[seg1 + e]; }
        __syncthreads();
        int token;
        const bool enough =   // (false only without top-k: the list does not hold top_p of the row)
            n <= 4 * PULSE_WAVE   // the usual case with top-k: a few dozen candidates, a few a lane
                ? finish_on_list<4>(list_i, list_x, n, by_k, k, use_p, p, whole, best, inv_t, uniform[r], best_i, token)
                : finish_on_list<LIST_PER_LANE>(list_i, list_x, n, by_k, k, use_p, p, whole, best, inv_t, uniform[r], best_i, token);
        if (lane == 0) {
            if (enough) out[r] = token;
            done[r] = enough ? 1 : 0;
        }
        return;
    }
    // a draw from the whole vocabulary: the chunk in which it falls, chunk masses in chunk order
    float total = 0.f;
    for (int c = lane; c < chunks; c += PULSE_WAVE) total += part_mass[c];
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) total += __shfl_xor(total, off, PULSE_WAVE);
    const float target = uniform[r] * total;
    float run = 0.f;
    int who = -1, last_chunk = -1;
    // (every lane the same few dozen additions; the masses come 64 at a time, one a lane, so that the additions do
    // not each wait for a trip to memory)
    for (int base = 0; base < chunks && who < 0; base += PULSE_WAVE) {
        const float mine = base + lane < chunks ? part_mass[base + lane] : 0.f;
        const int n = min(PULSE_WAVE, chunks - base);
        for (int j = 0; j < n; ++j) {
            const float m = __shfl(mine, j, PULSE_WAVE);
            if (m > 0.f) {
                last_chunk = base + j;
                if (target < run + m) { who = base + j; break; }
            }
            run += m;
        }
    }
    float rest = target - run;
    if (who < 0) {  // rounding left the target beyond the last chunk with mass: its last kept entry
        who = last_chunk;
        rest = INFINITY;
    }
    const RowView row = simple_row(logits, r, row_stride, vocab, penalty, seen_row, seen_masks, banned, mask_words);
    const int begin = who * SIMPLE_CHUNK, end = min(vocab, begin + SIMPLE_CHUNK);
    int last;
    const int e = wave_walk(begin, end, rest, [&](int i) {
        const float x = row.at(i);
        return x != -INFINITY ? expf((x - best) * inv_t) : 0.f;
    }, last);
    if (lane == 0) { out[r] = e >= 0 ? e : (last >= 0 ? last : best_i); done[r] = 1; }
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

// The same without a workspace argument: the chunk winners go through an array in the library's device image.
// In host code the array's name is only a stand-in for the symbol; its address on a device comes from
// hipGetSymbolAddress, once per device, and that pointer is what the kernels get.
static __device__ __align__(256) unsigned char argmax_static_scratch[PULSE_ARGMAX_STATIC_ENTRIES * 8];

namespace {
constexpr int STATIC_MAX_DEVICES = 64;
void* g_static_scratch[STATIC_MAX_DEVICES] = {};
std::mutex g_static_lock;
}  // namespace

extern "C" int pulse_argmax_static(const float* logits, int rows, int vocab, int64_t row_stride, int* out,
                                   hipStream_t stream) {
    PULSE_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax_static: bad sizes rows=%d V=%d", rows, vocab);
    PULSE_REQUIRE(rows < 65536, "argmax_static: at most 65535 rows");
    PULSE_REQUIRE(logits && out, "argmax_static: null pointer");
    const int chunks = pulse_argmax_chunks(vocab);
    PULSE_REQUIRE(static_cast<int64_t>(rows) * chunks <= PULSE_ARGMAX_STATIC_ENTRIES,
                  "argmax_static: %d rows x %d chunks of the vocabulary exceed the %d entries of the built-in scratch "
                  "array; use pulse_argmax with a workspace", rows, chunks, PULSE_ARGMAX_STATIC_ENTRIES);
    if (rows == 0) return 0;
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    PULSE_REQUIRE(err == hipSuccess, "argmax_static: hipGetDevice: %s", hipGetErrorString(err));
    PULSE_REQUIRE(device >= 0 && device < STATIC_MAX_DEVICES, "argmax_static: device %d is beyond the %d this entry "
                  "point keeps an address for", device, STATIC_MAX_DEVICES);
    void* base = nullptr;
    {
        std::lock_guard<std::mutex> hold(g_static_lock);
        if (!g_static_scratch[device]) {   // each GPU holds its own copy of the array at its own address
            void* found = nullptr;
            err = hipGetSymbolAddress(&found, HIP_SYMBOL(argmax_static_scratch));
            PULSE_REQUIRE(err == hipSuccess && found, "argmax_static: hipGetSymbolAddress on device %d: %s", device,
                          hipGetErrorString(err));
            g_static_scratch[device] = found;
        }
        base = g_static_scratch[device];
    }
    float* part_val = static_cast<float*>(base);
    int* part_idx = reinterpret_cast<int*>(static_cast<unsigned char*>(base) + PULSE_ARGMAX_STATIC_ENTRIES * 4);
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(chunks, rows), dim3(ARGMAX_THREADS), 0, stream, logits, vocab,
                       row_stride, 2048, part_val, part_idx);
    PULSE_LAUNCH_CHECK("argmax_static chunks");
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(rows), dim3(PULSE_WAVE), 0, stream, part_val, part_idx, chunks, out);
    PULSE_LAUNCH_CHECK("argmax_static merge");
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
                       temperature, top_k, top_p, uniform, penalty, seen_row, seen_masks, banned, mask_words, out,
                       static_cast<const int*>(nullptr));
    PULSE_LAUNCH_CHECK("sample");
    return 0;
}

// The same in chunks of the vocabulary with a workgroup each, which reads a row many times faster than the
// workgroup a row of pulse_sample does.  Greedy rows, rows that draw from the whole vocabulary at their temperature
// rows with top-k (and top-p on what it keeps) whose k is at most the number of chunks and rows with top-p alone whose
// top_p share lies in some hundreds of the largest logits are chosen by these kernels; rows that do not fit (many
// equal values around the k-th largest, a distribution too flat for top-p alone) by the kernel of pulse_sample behind
// them, which skips the rows that are done.  What a row's choice is does not depend on the
// other rows.  Scratch, with chunks = pulse_sample_chunks(vocab): part_max, part_mass (float32), part_idx, seg_n
// (int32) of rows * chunks entries; seg_i (int32), seg_x (float32) of rows * chunks * pulse_sample_segment()
// entries; done (int32) of rows entries.
extern "C" int pulse_sample_chunks(int vocab) { return (vocab + SIMPLE_CHUNK - 1) / SIMPLE_CHUNK; }
extern "C" int pulse_sample_segment() { return TOPK_SEGMENT; }

extern "C" int pulse_sample_chunked(const float* logits, int rows, int vocab, int64_t row_stride, const float* temperature,
                                    const int* top_k, const float* top_p, const float* uniform, const float* penalty,
                                    const int* seen_row, const uint32_t* seen_masks, const uint32_t* banned,
                                    int mask_words, float* part_max, int* part_idx, float* part_mass, int* seg_i,
                                    float* seg_x, int* seg_n, int* done, int* out, hipStream_t stream) {
    PULSE_REQUIRE(rows >= 0 && vocab > 0 && row_stride >= vocab, "sample_chunked: bad sizes rows=%d V=%d", rows, vocab);
    PULSE_REQUIRE(rows < 65536, "sample_chunked: at most 65535 rows");
    PULSE_REQUIRE(logits && out && part_max && part_idx && part_mass && seg_i && seg_x && seg_n && done,
                  "sample_chunked: null pointer");
    PULSE_REQUIRE(!temperature || uniform, "sample_chunked: temperature sampling needs uniform numbers");
    PULSE_REQUIRE((!seen_masks && !banned) || mask_words * 32 >= vocab, "sample_chunked: masks cover %d tokens, "
                  "vocabulary has %d", mask_words * 32, vocab);
    if (rows == 0) return 0;
    const int chunks = pulse_sample_chunks(vocab);
    hipLaunchKernelGGL(simple_max_kernel, dim3(chunks, rows), dim3(SIMPLE_THREADS), 0, stream, logits, vocab, row_stride,
                       penalty, seen_row, seen_masks, banned, mask_words, part_max, part_idx);
    PULSE_LAUNCH_CHECK("sample_chunked (maxima)");
    if (temperature) {
        hipLaunchKernelGGL(simple_mass_kernel, dim3(chunks, rows), dim3(SIMPLE_THREADS), 0, stream, logits, vocab,
                           row_stride, temperature, top_k, penalty, seen_row, seen_masks, banned, mask_words,
                           part_max, part_mass);
        PULSE_LAUNCH_CHECK("sample_chunked (masses)");
        if (top_k || top_p) {
            hipLaunchKernelGGL(topk_collect_kernel, dim3(chunks, rows), dim3(SIMPLE_THREADS), 0, stream, logits, vocab,
                               row_stride, temperature, top_k, top_p, penalty, seen_row, seen_masks, banned, mask_words,
                               part_max, seg_i, seg_x, seg_n);
            PULSE_LAUNCH_CHECK("sample_chunked (candidates)");
        }
    }
    hipLaunchKernelGGL(chunked_choose_kernel, dim3(rows), dim3(PULSE_WAVE), 0, stream, logits, vocab, row_stride,
                       temperature, top_k, top_p, uniform, penalty, seen_row, seen_masks, banned, mask_words, part_max,
                       part_idx, part_mass, seg_i, seg_x, seg_n, chunks, out, done);
    PULSE_LAUNCH_CHECK("sample_chunked (choice)");
    if (temperature && (top_k || top_p)) {   // (without them every row is done)
        hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, vocab, row_stride,
                           temperature, top_k, top_p, uniform, penalty, seen_row, seen_masks, banned, mask_words, out,
                           static_cast<const int*>(done));
        PULSE_LAUNCH_CHECK("sample_chunked (the rest)");
    }
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
