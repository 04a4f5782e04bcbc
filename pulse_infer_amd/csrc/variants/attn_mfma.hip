// Paged causal attention on the matrix cores for bfloat16, compiled for one
// head size (-DPULSE_HEAD_DIM=...).  The same kernel serves decoding and prompt
// portions.
//
// Work item: up to 16 "columns" that share one request and one kv head: the
// G = nq / nkv query heads of 16 / G' consecutive tokens (G' = G rounded up to
// a power of two; a decoded token is an item with one token).  A wavefront
// keeps everything transposed so that a column never leaves its lane group:
//
//   S^T[key, col] = K[key, :] . Q[col, :]      v_mfma_f32_16x16x32_bf16, A = K page rows, B = Q^T
//   P^T = exp2(S^T * scale*log2e - m[col])     running maximum per column, float32
//   O^T[ch, col] += V^T[ch, key] P^T[key, col]  A = V page rows (stored [channel][slot]), B = P^T
//
// Lane l supplies row l % 16 and the 8 contraction elements 8*(l/16).. of both
// operands, and receives rows 4*(l/16).. of column l % 16.  S^T comes out with
// keys 4*(l/16)+i per 16-key tile; two tiles give the 8 contraction elements of
// the second product in the order {tile0: 4g..4g+3, tile1: 4g..4g+3}, and V is
// loaded in that same order, so no data moves between lanes.
//
// The keys of an item are cut into splits of `split_size` keys (grid.z); the
// four wavefronts of a workgroup share a split's 32-key blocks and merge
// through LDS.  With one split the output is written directly, otherwise
// unnormalised partial results go to scratch and attn_mfma_reduce merges them.
// Scores, maxima, sums and accumulators are float32
// (reference formula: src/ops/kernels/cuda/paged_attention.cu:88-137).
#include "../common.h"

#include <math.h>

#ifndef PULSE_HEAD_DIM
#error "compile with -DPULSE_HEAD_DIM=<head size>"
#endif

namespace {

constexpr int D = PULSE_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 224, "head size must be a multiple of 16 up to 224 (the merge buffer must fit LDS)");
constexpr int NCHUNK = (D + 31) / 32;  // 32-wide slices of the q.k contraction
constexpr int NDT = D / 16;            // 16-channel tiles of the output
constexpr int WAVES = 4;
constexpr int BLOCK_KEYS = 32;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

struct MfmaArgs {
    const bf16_t* q;
    int64_t q_stride;
    bf16_t* out;
    int64_t o_stride;
    float* part_o;   // [T * nq, n_splits, D]
    float* part_ml;  // [T * nq, n_splits, 2]
    const bf16_t* kc;
    const bf16_t* vc;
    const int* positions;
    const int* token_entry;
    const int* block_table;
    const int* items;  // [n_items, 2]: first token row, number of tokens
    int bt_width;
    int nq, nkv, group;
    int gp;           // columns per token: the group size rounded up to a power of two, at most 16
    int head_chunks;  // ceil(group / 16)
    int page_size, num_pages;
    float scale_log2e;
    int window;
    int split_size;  // multiple of 32
    int n_splits;
};

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
}

__global__ __launch_bounds__(WAVES* PULSE_WAVE) void attn_mfma_kernel(MfmaArgs a) {
    __shared__ float s_m[WAVES][16];
    __shared__ float s_l[WAVES][16];
    __shared__ float s_o[WAVES][D][17];

    const int item = blockIdx.x;
    const int g = blockIdx.y / a.head_chunks;       // kv head
    const int chunk = blockIdx.y % a.head_chunks;   // which 16 heads of the group
    const int split = blockIdx.z;
    const int tid = threadIdx.x;
    const int wave = tid / PULSE_WAVE;
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;   // operand row / result column
    const int kg = lane / 16;  // contraction group / result row group

    const int row0 = a.items[2 * item];
    const int ntok = a.items[2 * item + 1];
    const int hi = a.positions[row0 + ntok - 1];    // last key any column of the item may see
    const int split_begin = split * a.split_size;
    if (split_begin > hi) return;                   // nothing here; the merge does not read this split
    const int split_end = min(split_begin + a.split_size, hi + 1);

    // this lane's column: a token of the item and a head of the group
    const int tc = r / a.gp;
    const int hc = r % a.gp + chunk * 16;
    const bool col_ok = tc < ntok && hc < a.group;
    const int col_row = row0 + (col_ok ? tc : 0);
    const int col_head = g * a.group + (col_ok ? hc : 0);
    const int pos_c = col_ok ? a.positions[col_row] : -1;
    const int lo_c = (a.window > 0 && pos_c - a.window + 1 > 0) ? pos_c - a.window + 1 : 0;
    // lowest key any column needs (the first token's window)
    const int pos_first = a.positions[row0];
    const int lo_item = (a.window > 0 && pos_first - a.window + 1 > 0) ? pos_first - a.window + 1 : 0;

    const int* bt = a.block_table + static_cast<int64_t>(a.token_entry[row0]) * a.bt_width;

    // Q^T operand: column r, contraction elements ch*32 + kg*8 ..
    bf16x8 bq[NCHUNK];
    {
        const bf16_t* qrow = a.q + static_cast<int64_t>(col_row) * a.q_stride + static_cast<int64_t>(col_head) * D;
#pragma unroll
        for (int ch = 0; ch < NCHUNK; ++ch) {
            const int off = ch * 32 + kg * 8;
            bq[ch] = (col_ok && off < D) ? *reinterpret_cast<const bf16x8*>(qrow + off) : zero8();
        }
    }

    f32x4 acc[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY;
    float l_part = 0.f;

    const int first_block = max(split_begin, lo_item) / BLOCK_KEYS;
    const int last_block = (split_end - 1) / BLOCK_KEYS;
    for (int b = first_block + wave; b <= last_block; b += WAVES) {
        const int j0 = b * BLOCK_KEYS;
        // pages of the two 16-key tiles (a tile never straddles pages: page_size % 16 == 0)
        int64_t kbase[2], vbase[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int jt = j0 + 16 * t;
            const int pi = jt / a.page_size;
            int page = (jt <= hi && pi < a.bt_width) ? bt[pi] : 0;
            page = (page >= 0 && page < a.num_pages) ? page : 0;  // masked keys may sit in pages given back
            const int slot0 = jt % a.page_size;
            const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
            kbase[t] = (pg * a.page_size + slot0) * D;
            vbase[t] = pg * D * a.page_size + slot0;
        }
        // S^T = K Q^T
        f32x4 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
            const bf16_t* krow = a.kc + kbase[t] + static_cast<int64_t>(r) * D;
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                const bf16x8 ak = off < D ? *reinterpret_cast<const bf16x8*>(krow + off) : zero8();
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak, bq[ch], s[t], 0, 0, 0);
            }
        }
        // V^T operands: channel row dt*16 + r, keys {tile0: 4kg.., tile1: 4kg..}
        bf16x8 av[NDT];
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            const int64_t ch_off = static_cast<int64_t>(dt * 16 + r) * a.page_size + 4 * kg;
            const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(a.vc + vbase[0] + ch_off);
            const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(a.vc + vbase[1] + ch_off);
            av[dt] = bf16x8{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
        }
        // scores of this lane: keys j0 + 16t + 4kg + i of column r
        const bool needs_mask = (j0 + BLOCK_KEYS - 1 > hi) || (j0 < lo_item + 0) || (a.window > 0) || (ntok > 1) ||
                                (j0 < split_begin) || (j0 + BLOCK_KEYS > split_end);
        float p[2][4];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + 16 * t + 4 * kg + i;
                float v = s[t][i] * a.scale_log2e;
                if (needs_mask && !(j <= pos_c && j >= lo_c && j >= split_begin && j < split_end)) v = -INFINITY;
                if (!col_ok) v = -INFINITY;
                p[t][i] = v;
                mx = fmaxf(mx, v);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, PULSE_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, PULSE_WAVE));
        const float m_new = fmaxf(m, mx);
        const float alpha = (m_new == -INFINITY) ? 1.f : exp2f(m - m_new);
        float psum = 0.f;
        bf16x8 pb;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float e = (p[t][i] == -INFINITY) ? 0.f : exp2f(p[t][i] - m_new);
                psum += e;
                pb[4 * t + i] = (__bf16)e;
            }
        l_part = l_part * alpha + psum;
        m = m_new;
        if (needs_mask) {
            // stale values under masked keys must not reach the sum, not even as 0 * (inf or nan)
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int j = j0 + 16 * (e / 4) + 4 * kg + (e % 4);
                    if (j > hi || j < lo_item) av[dt][e] = (__bf16)0.0f;
                }
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            acc[dt] = acc[dt] * alpha;
            acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[dt], pb, acc[dt], 0, 0, 0);
        }
    }

    // the column's sum sits in four lanes
    l_part += __shfl_xor(l_part, 16, PULSE_WAVE);
    l_part += __shfl_xor(l_part, 32, PULSE_WAVE);
    if (kg == 0) {
        s_m[wave][r] = m;
        s_l[wave][r] = l_part;
    }
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_o[wave][dt * 16 + 4 * kg + i][r] = acc[dt][i];
    __syncthreads();

    // merge the four wavefronts; thread -> column tid / 16, channels tid % 16 + 16 k
    const int c = tid / 16;
    const int dd = tid % 16;
    const int tc2 = c / a.gp;
    const int hc2 = c % a.gp + chunk * 16;
    if (!(tc2 < ntok && hc2 < a.group)) return;
    float mm = s_m[0][c];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) mm = fmaxf(mm, s_m[w][c]);
    float wgt[WAVES];
    float ll = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        wgt[w] = (s_m[w][c] == -INFINITY) ? 0.f : exp2f(s_m[w][c] - mm);
        ll += wgt[w] * s_l[w][c];
    }
    const int64_t row = row0 + tc2;
    const int head = g * a.group + hc2;
    if (a.n_splits == 1) {
        const float inv = ll > 0.f ? 1.0f / ll : 0.f;
        bf16_t* dst = a.out + row * a.o_stride + static_cast<int64_t>(head) * D;
        for (int ch = dd; ch < D; ch += 16) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += wgt[w] * s_o[w][ch][c];
            dst[ch] = f32_to_bf16(v * inv);
        }
    } else {
        const int64_t slot = (row * a.nq + head) * a.n_splits + split;
        float* dst = a.part_o + slot * D;
        for (int ch = dd; ch < D; ch += 16) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += wgt[w] * s_o[w][ch][c];
            dst[ch] = v;
        }
        if (dd == 0) {
            a.part_ml[2 * slot] = mm;
            a.part_ml[2 * slot + 1] = ll;
        }
    }
}

// out[row, head, :] = sum_z w_z o_z / sum_z w_z l_z with w_z = exp2(m_z - max m), over the splits that hold keys of
// the row.  One workgroup per (row, head); the splits' (m, l) pairs go through LDS so that the loads overlap.
constexpr int MAX_SPLITS = 1024;

__global__ __launch_bounds__(128) void attn_mfma_reduce_kernel(const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml,
                                                               const int* __restrict__ positions, bf16_t* __restrict__ out,
                                                               int64_t o_stride, int nq, int n_splits, int split_size) {
    __shared__ float s_w[MAX_SPLITS];
    __shared__ float s_l[MAX_SPLITS];
    const int64_t row = blockIdx.x;
    const int head = blockIdx.y;
    const int valid = min(n_splits, positions[row] / split_size + 1);
    const int64_t base = (row * nq + head) * n_splits;
    for (int z = threadIdx.x; z < valid; z += blockDim.x) {
        s_w[z] = part_ml[2 * (base + z)];
        s_l[z] = part_ml[2 * (base + z) + 1];
    }
    __syncthreads();
    float mm = -INFINITY;
    for (int z = 0; z < valid; ++z) mm = fmaxf(mm, s_w[z]);
    float ll = 0.f;
    for (int z = 0; z < valid; ++z) ll += (s_w[z] == -INFINITY ? 0.f : exp2f(s_w[z] - mm)) * s_l[z];
    const float inv = ll > 0.f ? 1.0f / ll : 0.f;
    bf16_t* dst = out + row * o_stride + static_cast<int64_t>(head) * D;
    for (int ch = threadIdx.x; ch < D; ch += blockDim.x) {
        float v = 0.f;
#pragma unroll 4
        for (int z = 0; z < valid; ++z) {
            const float wz = s_w[z] == -INFINITY ? 0.f : exp2f(s_w[z] - mm);
            v += wz * part_o[(base + z) * D + ch];
        }
        dst[ch] = f32_to_bf16(v * inv);
    }
}

}  // namespace

extern "C" int pulse_attn_mfma_head_dim() { return D; }

// Scratch needed for `tokens` rows cut into `n_splits`: floats of part_o and of part_ml.
extern "C" int pulse_attn_mfma(const void* q, int64_t q_stride, void* out, int64_t o_stride, const void* kcache,
                               const void* vcache, const int* positions, const int* token_entry,
                               const int* block_table, int bt_width, const int* items, int n_items, int tokens, int nq,
                               int nkv, int page_size, int num_pages, float scale, int window, int split_size,
                               int n_splits, int max_context, float* part_o, float* part_ml, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && n_items >= 0 && nq > 0 && nkv > 0, "attn_mfma: bad sizes");
    PULSE_REQUIRE(nq % nkv == 0, "attn_mfma: %d query heads are not a multiple of %d kv heads", nq, nkv);
    PULSE_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_mfma: page size %d must be a multiple of 16", page_size);
    PULSE_REQUIRE(num_pages > 0 && bt_width > 0, "attn_mfma: bad cache geometry");
    PULSE_REQUIRE(q_stride % 8 == 0 && q_stride >= static_cast<int64_t>(nq) * D && o_stride >= static_cast<int64_t>(nq) * D,
                  "attn_mfma: row strides must cover the heads and keep 16-byte alignment");
    PULSE_REQUIRE((reinterpret_cast<uintptr_t>(q) % 16) == 0 && (reinterpret_cast<uintptr_t>(kcache) % 16) == 0 &&
                  (reinterpret_cast<uintptr_t>(vcache) % 16) == 0, "attn_mfma: pointers must be 16-byte aligned");
    PULSE_REQUIRE(window >= 0 && n_splits >= 1 && split_size >= BLOCK_KEYS && split_size % BLOCK_KEYS == 0,
                  "attn_mfma: split size %d must be a positive multiple of %d", split_size, BLOCK_KEYS);
    PULSE_REQUIRE(static_cast<int64_t>(n_splits) * split_size >= max_context,
                  "attn_mfma: %d splits of %d keys do not cover a context of %d", n_splits, split_size, max_context);
    PULSE_REQUIRE(n_splits == 1 || (part_o && part_ml), "attn_mfma: scratch is missing");
    PULSE_REQUIRE(n_splits <= MAX_SPLITS, "attn_mfma: at most %d splits, got %d", MAX_SPLITS, n_splits);
    PULSE_REQUIRE(n_splits < 65536 && static_cast<int64_t>(nkv) * ((nq / nkv + 15) / 16) < 65536, "attn_mfma: grid too large");
    PULSE_REQUIRE(q && out && kcache && vcache && positions && token_entry && block_table && items, "attn_mfma: null pointer");
    if (tokens == 0 || n_items == 0) return 0;
    const int group = nq / nkv;
    int gp = 1;
    while (gp < group && gp < 16) gp *= 2;
    MfmaArgs a;
    a.q = static_cast<const bf16_t*>(q); a.q_stride = q_stride;
    a.out = static_cast<bf16_t*>(out); a.o_stride = o_stride;
    a.part_o = part_o; a.part_ml = part_ml;
    a.kc = static_cast<const bf16_t*>(kcache); a.vc = static_cast<const bf16_t*>(vcache);
    a.positions = positions; a.token_entry = token_entry; a.block_table = block_table; a.items = items;
    a.bt_width = bt_width; a.nq = nq; a.nkv = nkv; a.group = group; a.gp = gp; a.head_chunks = (group + 15) / 16;
    a.page_size = page_size; a.num_pages = num_pages;
    a.scale_log2e = scale * 1.4426950408889634f;
    a.window = window; a.split_size = split_size; a.n_splits = n_splits;
    hipLaunchKernelGGL(attn_mfma_kernel, dim3(n_items, nkv * a.head_chunks, n_splits), dim3(WAVES * PULSE_WAVE), 0,
                       stream, a);
    PULSE_LAUNCH_CHECK("attn_mfma");
    if (n_splits > 1) {
        hipLaunchKernelGGL(attn_mfma_reduce_kernel, dim3(tokens, nq), dim3(128), 0, stream, part_o, part_ml, positions,
                           a.out, o_stride, nq, n_splits, split_size);
        PULSE_LAUNCH_CHECK("attn_mfma_reduce");
    }
    return 0;
}

// Columns per token and tokens per item for a group size: the host builds its item list with these.
extern "C" int pulse_attn_mfma_tokens_per_item(int group) {
    int gp = 1;
    while (gp < group && gp < 16) gp *= 2;
    return 16 / gp;
}
