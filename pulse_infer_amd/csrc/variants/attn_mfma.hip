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
// Column tiles a wavefront takes in the prompt-portion kernel: two while the accumulators of both fit the registers.
#define PULSE_WIDE (PULSE_HEAD_DIM == 32 || PULSE_HEAD_DIM == 64 || PULSE_HEAD_DIM == 128)
#ifndef PULSE_WIDE_CT
#define PULSE_WIDE_CT 2
#endif
constexpr int WIDE_NW = 4;   // wavefronts of the wide prompt-portion kernel
constexpr int WIDE_CT = PULSE_WIDE_CT;   // column tiles each takes
constexpr int PREFILL_TILES = PULSE_WIDE ? WIDE_CT : 1;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// The operands of one 32-key block as they come from memory.
struct BlockRegs {
    u32x4 k[2][NCHUNK];  // tile, 32-wide slice of the head: 8 bfloat16 of key row r
    u32x2 v[2][NDT];     // tile, 16-channel tile: 4 bfloat16 (keys 4kg..4kg+3) of channel row r
};

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
    const int* block_table;
    const int* items;  // [n_items, 4]: first token row, number of tokens, row of the block table, 0; or null: item i
                       // is token i alone with row i of the block table (a step of decoded tokens in the order of
                       // its requests), which saves every workgroup a trip to memory before its first load of keys
    int bt_width;
    int n_items;
    int nq, nkv, group;
    int gp;           // columns per token: the group size rounded up to a power of two, at most 16
    int head_chunks;  // ceil(group / 16)
    int page_size, num_pages;
    int page_shift;   // log2(page_size) when it is a power of two, else -1
    float scale_log2e;
    int window;
    int split_size;  // multiple of 32
    int n_splits;
    // The longest context of the step as it is now, or null.  The launch (and a recording of it) is made for contexts
    // up to n_splits * split_size; with this the kernel of decoded tokens cuts the keys that are there into n_splits
    // even splits instead (see live_split_size), so that no split stands empty while another walks its full length.
    const int* live_context;
    // Or null: the step's plan (made by attn_plan_kernel from the contexts as they are now), which takes the place
    // of the even cut above.  plan[0] (item, split) pairs in the order the workgroups take them, pair k as
    // plan[1 + k] = item * n_splits + split (workgroups beyond the count leave at once); behind the n_items *
    // n_splits places for pairs, every item's own split size: its keys are cut into as many splits as its length
    // asks for, an item of one split is finished by its workgroup, and no workgroup stands empty.
    const int* plan;
    // Only for the kernel that prepares q and the step's own key itself (decoded tokens): then q points at the raw
    // projection output [T, (nq + 2 nkv) D] (q heads, k heads, v heads), as the kernel of qk_rope_kv.hip takes it.
    const bf16_t* q_w;     // per-head RMSNorm weights [D], or null for no norm
    const bf16_t* k_w;
    const float* cos_t;    // [T, rotary_dim / 2], or null for no rotation
    const float* sin_t;
    float eps;
    int rotary_dim;        // multiple of 8
    int pairing;           // 0: (2i, 2i+1)   1: (i, i + rotary_dim / 2), rotary_dim a multiple of 64
    int new_key;           // 1: the token's key and value are prepared, used and written to their page here
};

// The split size for a step whose longest context is `live` (at most n_splits * split_size, what the launch was made
// for): the keys cut evenly into the launch's number of splits, in whole 32-key blocks, never more than split_size.
__device__ __forceinline__ int live_split_size(int live, int n_splits, int split_size) {
    const int even = ((max(live, 1) + n_splits - 1) / n_splits + 31) / 32 * 32;
    return min(split_size, even);
}

// A value that is the same in every lane of the wavefront, said so to the compiler: what depends on it becomes
// scalar work and uniform branches.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// Page index and slot of a key: a shift when the page size is a power of two (divisions by a run-time
// number cost dozens of scalar instructions in the inner loop).
__device__ __forceinline__ void page_of(int j, int page_size, int page_shift, int& pi, int& slot) {
    if (page_shift >= 0) {
        pi = j >> page_shift;
        slot = j & (page_size - 1);
    } else {
        pi = j / page_size;
        slot = j - pi * page_size;
    }
}

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
}

// What the preparation of a head needs besides the head: norm weight, cos and sin of this lane's slices (for pairs
// (2i, 2i+1) the four angles of a slice, for pairs (i, i + rotary_dim / 2) the eight of a slice of the first half).
struct HeadTables {
    bf16x8 w[NCHUNK];
    float cs[NCHUNK][8];
    float sn[NCHUNK][8];
};

// Rotation of the pairs (i, i + 32 SHIFT): the partner slice lies SHIFT chunks further on, in the same lane.
template <int SHIFT>
__device__ __forceinline__ void rotate_halves(float (&f)[NCHUNK][8], const HeadTables& tb) {
#pragma unroll
    for (int ch = 0; ch < SHIFT; ++ch) {
        if (ch + SHIFT >= NCHUNK) continue;
        constexpr int LAST = NCHUNK - 1;
        const int c2 = ch + SHIFT < NCHUNK ? ch + SHIFT : LAST;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float va = f[ch][e], vb = f[c2][e];
            f[ch][e] = va * tb.cs[ch][e] - vb * tb.sn[ch][e];
            f[c2][e] = va * tb.sn[ch][e] + vb * tb.cs[ch][e];
        }
    }
}

// Per-head RMSNorm and rotation of one head whose 8-element slices ch*32 + kg*8.. sit in the four lanes kg = 0..3
// of a column, with the arithmetic of qk_rope_kv.hip: float32, (x * inv) * w, then the rotation, one rounding.
__device__ __forceinline__ void prepare_head(bf16x8 (&x)[NCHUNK], const HeadTables& tb, bool normed, bool rotated,
                                             float eps, int rot, int pairing, int kg) {
    float f[NCHUNK][8];
    float ss = 0.f;
#pragma unroll
    for (int ch = 0; ch < NCHUNK; ++ch)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            f[ch][e] = static_cast<float>(x[ch][e]);
            ss += f[ch][e] * f[ch][e];
        }
    if (normed) {
        ss += __shfl_xor(ss, 16, PULSE_WAVE);
        ss += __shfl_xor(ss, 32, PULSE_WAVE);
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(D) + eps);
#pragma unroll
        for (int ch = 0; ch < NCHUNK; ++ch)
#pragma unroll
            for (int e = 0; e < 8; ++e) f[ch][e] = f[ch][e] * inv * static_cast<float>(tb.w[ch][e]);
    }
    if (rotated) {
        if (pairing == 0) {
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch)
                if (ch * 32 + kg * 8 < rot) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float va = f[ch][2 * i], vb = f[ch][2 * i + 1];
                        f[ch][2 * i] = va * tb.cs[ch][i] - vb * tb.sn[ch][i];
                        f[ch][2 * i + 1] = va * tb.sn[ch][i] + vb * tb.cs[ch][i];
                    }
                }
        } else {
            switch (rot / 64) {
                case 1: rotate_halves<1>(f, tb); break;
                case 2: rotate_halves<2>(f, tb); break;
                case 3: rotate_halves<3>(f, tb); break;
                default: break;
            }
        }
    }
#pragma unroll
    for (int ch = 0; ch < NCHUNK; ++ch)
#pragma unroll
        for (int e = 0; e < 8; ++e) x[ch][e] = (__bf16)f[ch][e];
}

// two wavefronts a SIMD (256 registers each) where the head size lets the two register sets fit
#if PULSE_HEAD_DIM <= 128
#define PULSE_ATTN_WAVES_PER_EU __attribute__((amdgpu_waves_per_eu(2)))
#else
#define PULSE_ATTN_WAVES_PER_EU
#endif

// FUSED: the items are decoded tokens (one token each) whose q, and whose own key and value if a.new_key, are still
// raw in the projection output.  Every workgroup prepares its q heads itself; the workgroup whose split holds the
// token's position also prepares the token's key, puts key and value into the registers of the block they belong
// to (their page is written from here and never read back), so that the launch before this one is saved.
template <bool FUSED>
__global__ __launch_bounds__(WAVES* PULSE_WAVE) PULSE_ATTN_WAVES_PER_EU void attn_mfma_kernel(MfmaArgs a) {
    __shared__ float s_m[WAVES][16];
    __shared__ float s_l[WAVES][16];
    __shared__ float s_o[WAVES][D][17];

    // Workgroups that follow each other in the grid go to different XCDs, each with its own L2 and its own share of
    // the way to memory (about an eighth of the chip's rate), and inside an XCD to different compute units, each of
    // which reads at about 32 GB/s at most in this kernel.  So the kv heads of an item follow each other, then its
    // splits, then the items: a request with a long context among short ones is then read through every XCD and by
    // as many compute units as it has workgroups.
    const int heads = a.nkv * a.head_chunks;
    const int hy = blockIdx.x % heads;
    int split = (blockIdx.x / heads) % a.n_splits;
    int item = blockIdx.x / heads / a.n_splits;
    if (a.plan) {
        const int k = blockIdx.x / heads;
        if (k >= a.plan[0]) return;
        const int s = a.plan[1 + k];
        item = s / a.n_splits;
        split = s % a.n_splits;
    }
    const int g = hy / a.head_chunks;       // kv head
    const int chunk = hy % a.head_chunks;   // which 16 heads of the group
    const int tid = threadIdx.x;
    const int wave = uniform(tid / PULSE_WAVE);   // the same in every lane: block numbers and pages become scalar work
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;   // operand row / result column
    const int kg = lane / 16;  // contraction group / result row group

    // Everything the first loads of keys need comes with the item (the block table's row too), so that the chain of
    // dependent trips to memory before a workgroup streams is item -> block table -> keys.  The positions (which only
    // decide masks and the end of the walk) and q travel at the same time.
    const bool listed = a.items != nullptr;
    const int row0 = listed ? a.items[4 * item] : item;
    const int ntok = listed ? a.items[4 * item + 1] : 1;
    const int* bt = a.block_table + static_cast<int64_t>(listed ? a.items[4 * item + 2] : item) * a.bt_width;
    const int hi = a.positions[row0 + ntok - 1];    // last key any column of the item may see
    const int split_size = a.plan ? a.plan[1 + a.n_items * a.n_splits + item]
                           : (a.live_context && a.n_splits > 1)
                               ? live_split_size(uniform(*a.live_context), a.n_splits, a.split_size) : a.split_size;
    const int split_begin = split * split_size;
    int split_end = 0;                              // set once hi has arrived

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

    // Q^T operand: column r, contraction elements ch*32 + kg*8 ..; loaded below, after the first keys are asked for
    bf16x8 bq[NCHUNK];
    bf16x8 knew[NCHUNK];   // FUSED: slice kg of the token's own key, the same in the 16 lanes of a kg
    bf16x8 kwt[NCHUNK];    // and of the key norm's weight
    constexpr int VPL = (D + PULSE_WAVE - 1) / PULSE_WAVE;
    bf16_t vown[VPL];      // FUSED: channels lane, lane + 64, .. of the token's own value
    int own_page = -1;     // FUSED: the page the token's key and value go to (asked for early, used at the end)
    HeadTables tb;
    auto load_q = [&]() {
        const bf16_t* qrow = a.q + static_cast<int64_t>(col_row) * a.q_stride + static_cast<int64_t>(col_head) * D;
#pragma unroll
        for (int ch = 0; ch < NCHUNK; ++ch) {
            const int off = ch * 32 + kg * 8;
            bq[ch] = (col_ok && off < D) ? *reinterpret_cast<const bf16x8*>(qrow + off) : zero8();
        }
        if (FUSED) {
            // everything the preparation needs is asked for here, behind the first keys: the raw key of the token,
            // the norm weights' slices, the slices of the token's cos and sin rows
            const bf16_t* krow = a.q + static_cast<int64_t>(row0) * a.q_stride + static_cast<int64_t>(a.nq + g) * D;
            const int half = a.rotary_dim / 2;
            const float* cos_row = a.cos_t ? a.cos_t + static_cast<int64_t>(row0) * half : nullptr;
            const float* sin_row = a.sin_t ? a.sin_t + static_cast<int64_t>(row0) * half : nullptr;
            const bf16_t* vraw = a.q + static_cast<int64_t>(row0) * a.q_stride + static_cast<int64_t>(a.nq + a.nkv + g) * D;
#pragma unroll
            for (int i = 0; i < VPL; ++i) vown[i] = (a.new_key && lane + i * PULSE_WAVE < D) ? vraw[lane + i * PULSE_WAVE] : 0;
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                knew[ch] = (a.new_key && off < D) ? *reinterpret_cast<const bf16x8*>(krow + off) : zero8();
                tb.w[ch] = (a.q_w && off < D) ? *reinterpret_cast<const bf16x8*>(a.q_w + off) : zero8();
                kwt[ch] = (a.new_key && a.k_w && off < D) ? *reinterpret_cast<const bf16x8*>(a.k_w + off) : zero8();
                // pairs (2i, 2i+1): the slice's four angles; pairs (i, i + half): the eight of a slice of the first half
                f32x4 c0 = {1.f, 1.f, 1.f, 1.f}, c1 = c0, s0 = {0.f, 0.f, 0.f, 0.f}, s1 = s0;
                if (cos_row && off < (a.pairing == 0 ? a.rotary_dim : half)) {
                    const int at = a.pairing == 0 ? off / 2 : off;
                    c0 = *reinterpret_cast<const f32x4*>(cos_row + at);
                    s0 = *reinterpret_cast<const f32x4*>(sin_row + at);
                    if (a.pairing != 0) {
                        c1 = *reinterpret_cast<const f32x4*>(cos_row + at + 4);
                        s1 = *reinterpret_cast<const f32x4*>(sin_row + at + 4);
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    tb.cs[ch][i] = c0[i]; tb.cs[ch][4 + i] = c1[i];
                    tb.sn[ch][i] = s0[i]; tb.sn[ch][4 + i] = s1[i];
                }
            }
        }
    };
    // FUSED: the token's key and value wait in LDS, a copy for each wavefront (so that no barrier is needed), until
    // the block they belong to is computed.
    __shared__ u32x4 s_newk[FUSED ? WAVES : 1][D / 8];
    __shared__ bf16_t s_newv[FUSED ? WAVES : 1][D];
    u32x4* stash_k = s_newk[FUSED ? wave : 0];
    bf16_t* stash_v = s_newv[FUSED ? wave : 0];
    auto prepare = [&](bool own_key) {
        prepare_head(bq, tb, a.q_w != nullptr, a.cos_t != nullptr, a.eps, a.rotary_dim, a.pairing, kg);
        if (!col_ok) {
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) bq[ch] = zero8();
        }
        if (!own_key) return;
        // the key's norm weight takes the place of q's; cos and sin are the token's for both
#pragma unroll
        for (int ch = 0; ch < NCHUNK; ++ch) tb.w[ch] = kwt[ch];
        prepare_head(knew, tb, a.k_w != nullptr, a.cos_t != nullptr, a.eps, a.rotary_dim, a.pairing, kg);
        if (r == 0) {
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                if (off < D) stash_k[off / 8] = __builtin_bit_cast(u32x4, knew[ch]);
            }
        }
#pragma unroll
        for (int i = 0; i < VPL; ++i)
            if (lane + i * PULSE_WAVE < D) stash_v[lane + i * PULSE_WAVE] = vown[i];
        // where key and value go, for the steps to come: asked for now, written when the walk over the keys is over
        int pi, slot;
        page_of(hi, a.page_size, a.page_shift, pi, slot);
        own_page = pi < a.bt_width ? bt[pi] : -1;
    };
    // FUSED: the first wavefront of the split that holds the token writes its key and value to their page
    auto store_own = [&]() {
        if (wave != 0 || own_page < 0 || own_page >= a.num_pages) return;
        int pi, slot;
        page_of(hi, a.page_size, a.page_shift, pi, slot);
        const int64_t pg = static_cast<int64_t>(own_page) * a.nkv + g;
        bf16_t* kdst = const_cast<bf16_t*>(a.kc) + (pg * a.page_size + slot) * D;
        bf16_t* vdst = const_cast<bf16_t*>(a.vc) + pg * D * a.page_size + slot;
        if (r == 0) {
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                if (off < D) *reinterpret_cast<u32x4*>(kdst + off) = stash_k[off / 8];
            }
        }
        for (int c = lane; c < D; c += PULSE_WAVE) vdst[static_cast<int64_t>(c) * a.page_size] = stash_v[c];
    };
    // FUSED: key `hi` of block `b` comes from the stash, not from its page
    auto patch = [&](BlockRegs& x) {
        const int tpos = (hi % BLOCK_KEYS) / 16;
        const int rpos = hi % 16;
        const int word = (hi % 4) / 2;
        const uint32_t sh = (hi % 2) * 16;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            if (t != tpos) continue;
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                if (off < D && r == rpos) x.k[t][ch] = stash_k[off / 8];
            }
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const uint32_t v = stash_v[dt * 16 + r];
                if (kg == rpos / 4) {
                    const uint32_t old = word == 0 ? x.v[t][dt][0] : x.v[t][dt][1];
                    const uint32_t neu = (old & ~(0xffffu << sh)) | (v << sh);
                    if (word == 0) x.v[t][dt][0] = neu;
                    else x.v[t][dt][1] = neu;
                }
            }
        }
    };

    f32x4 acc[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY;
    float l_part = 0.f;

    // The loads of a 32-key block come in two steps, each issued whatever the block (a load under a condition would
    // keep the compiler from counting the loads in flight: it would then wait for all of them, the next block's
    // too, before it touches this block's).  First the pages of the block's two 16-key tiles (a tile never straddles
    // pages: page_size % 16 == 0) from the block table, an iteration before they are needed; an index beyond the
    // table reads its last entry, which is not used then.
    struct BlockPages { int page[2]; };
    auto load_pages = [&](int b) {
        BlockPages p;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            int pi, slot0;
            page_of(b * BLOCK_KEYS + 16 * t, a.page_size, a.page_shift, pi, slot0);
            p.page[t] = bt[min(pi, a.bt_width - 1)];
        }
        return p;
    };
    // Then every load of the block (nontemporal: a step reads a request's keys and values once): K rows of the two
    // tiles and V rows in the order {tile0: 4kg.., tile1: 4kg..}.
    // Nothing is done to the values here.  A page that the table does not hold (-1, or beyond its width) reads
    // page 0: those keys are masked.
    auto load_block = [&](int b, const BlockPages& pages, BlockRegs& x) {
        const int j0 = b * BLOCK_KEYS;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int jt = j0 + 16 * t;
            int pi, slot0;
            page_of(jt, a.page_size, a.page_shift, pi, slot0);
            int page = pi < a.bt_width ? pages.page[t] : 0;
            page = (page >= 0 && page < a.num_pages) ? page : 0;  // masked keys may sit in pages given back
            const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
            const bf16_t* krow = a.kc + (pg * a.page_size + slot0 + r) * D;
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                x.k[t][ch] = off < D ? __builtin_bit_cast(u32x4, stream_load16(krow + off)) : u32x4{0u, 0u, 0u, 0u};
            }
            const bf16_t* vrow = a.vc + pg * D * a.page_size + slot0 + 4 * kg + static_cast<int64_t>(r) * a.page_size;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                x.v[t][dt] = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(vrow + static_cast<int64_t>(dt) * 16 * a.page_size));
        }
    };

    auto compute_block = [&](int b, const BlockRegs& x) {
        const int j0 = b * BLOCK_KEYS;
        // S^T = K Q^T
        f32x4 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch)
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x.k[t][ch]), bq[ch], s[t], 0, 0, 0);
        }
        // scores of this lane: keys j0 + 16t + 4kg + i of column r
        const bool needs_mask = (j0 + BLOCK_KEYS - 1 > hi) || (j0 < lo_item) || (a.window > 0) || (ntok > 1) ||
                                (j0 < split_begin) || (j0 + BLOCK_KEYS > split_end);
        float p[2][4];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = j0 + 16 * t + 4 * kg + i;
                float v = s[t][i] * a.scale_log2e;
                const bool seen = !needs_mask || (j <= pos_c && j >= lo_c && j >= split_begin && j < split_end);
                v = (seen && col_ok) ? v : -INFINITY;
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
        // Stale values under keys that no column of the item may see must not reach the sum, not even as
        // 0 * (inf or nan): they are cleared by bit masks, one per pair of keys.
        uint32_t keep[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
                const int j = j0 + 16 * t + 4 * kg + 2 * h2;
                const bool lo_ok = !needs_mask || (j <= hi && j >= lo_item);
                const bool hi_ok = !needs_mask || (j + 1 <= hi && j + 1 >= lo_item);
                keep[t][h2] = (lo_ok ? 0x0000ffffu : 0u) | (hi_ok ? 0xffff0000u : 0u);
            }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            const u32x4 words = {x.v[0][dt][0] & keep[0][0], x.v[0][dt][1] & keep[0][1],
                                 x.v[1][dt][0] & keep[1][0], x.v[1][dt][1] & keep[1][1]};
            acc[dt] = acc[dt] * alpha;
            acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, words), pb, acc[dt], 0, 0, 0);
        }
    };

    // Two register sets in turn: the next block's loads are in flight while this block is computed, and the pages
    // of the block after that are on their way.  Behind a wavefront's last block the "next" block is the one in hand
    // once more (its lines are in the cache; nothing uses the result).  Without a window the first block is known
    // from the split alone: its loads go out before the positions have arrived.
    {
        BlockRegs xa, xb;
        const bool early = a.window == 0;
        int b = split_begin / BLOCK_KEYS + wave;
        // Results come back in the order asked for.  Plain: the keys first, q behind them (it is needed only when
        // the first keys are there).  FUSED: q, the token's raw key and what their preparation needs go out between
        // the first block's pages and its keys, which wait for the pages anyway: they arrive a trip before the keys,
        // and the preparation runs while the keys are on their way instead of after they have come.
        const BlockPages p0 = load_pages(b);
        if (FUSED) load_q();
        if (early && b <= (split_begin + split_size - 1) / BLOCK_KEYS) load_block(b, p0, xa);
        if (!FUSED) load_q();
        if (split_begin > hi) return;                   // nothing here; the merge does not read this split
        split_end = min(split_begin + split_size, hi + 1);
        const int first_block = max(split_begin, lo_item) / BLOCK_KEYS;
        const int last_block = (split_end - 1) / BLOCK_KEYS;
        // FUSED: the split that holds the token's position (the last one with keys) has its key to prepare
        const bool own_key = FUSED && a.new_key && hi < split_begin + split_size;
        const int own_block = own_key ? hi / BLOCK_KEYS : -1;
        auto after = [&](int blk) { return blk + WAVES <= last_block ? blk + WAVES : blk; };
        BlockPages pa = load_pages(after(b)), pb;       // (with a window b moves below; the pages are asked for again)
        if (FUSED) prepare(own_key);
        if (!early) {
            b = first_block + wave;
            if (b <= last_block) load_block(b, load_pages(b), xa);
            pa = load_pages(after(b));
        }
        while (b <= last_block) {
            int nb = after(b);
            pb = load_pages(after(nb));
            load_block(nb, pa, xb);
            if (FUSED && b == own_block) patch(xa);
            compute_block(b, xa);
            b += WAVES;
            if (b > last_block) break;
            nb = after(b);
            pa = load_pages(after(nb));
            load_block(nb, pb, xa);
            if (FUSED && b == own_block) patch(xb);
            compute_block(b, xb);
            b += WAVES;
        }
        if (FUSED && own_key) store_own();
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
    if (a.n_splits == 1 || (a.plan && hi < split_size)) {   // the only split of its item: nothing to merge
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

// ---------------------------------------------------------------------------------------------------------
// Prompt portions: one workgroup per (item, kv head, chunk of 16 heads); its four wavefronts take consecutive
// sub-items of `per` tokens (16 columns each) and walk the keys together.  Every 32-key block of K and V is copied
// from its pages into LDS once for all four (two stages, so the next block's loads are in flight while this one
// is computed), and each wavefront reads its matrix-core operands from there.  No split: a wavefront sees all its
// keys, so it normalises and writes its columns itself.
constexpr int KPAD = 8;                    // bfloat16 of padding a key row: 16-byte reads of 16 rows hit 16 bank groups
constexpr int KROW = D + KPAD;
constexpr int STAGE_K = BLOCK_KEYS * KROW;  // bfloat16 elements
// V in LDS, in 8-byte words (4 keys of one channel): [tile][16-channel tile][key group kg][channel row r], padded to
// 17 words a key group, so that the 16 lanes of one key group read 128 contiguous bytes (no bank conflict).
constexpr int VGROUP = 17;
constexpr int STAGE_V = 2 * NDT * 4 * VGROUP * 4;  // bfloat16 elements

__global__ __launch_bounds__(WAVES* PULSE_WAVE) PULSE_ATTN_WAVES_PER_EU void attn_prefill_kernel(MfmaArgs a, int per) {
    __shared__ __attribute__((aligned(16))) bf16_t s_k[2][STAGE_K];
    __shared__ __attribute__((aligned(16))) bf16_t s_v[2][STAGE_V];

    const int item = blockIdx.x;
    const int g = blockIdx.y / a.head_chunks;
    const int chunk = blockIdx.y % a.head_chunks;
    const int tid = threadIdx.x;
    const int wave = uniform(tid / PULSE_WAVE);
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;

    const int row0 = uniform(a.items[4 * item]);
    const int ntok = uniform(a.items[4 * item + 1]);         // at most WAVES * per
    const int hi = uniform(a.positions[row0 + ntok - 1]);    // last key of the workgroup
    const int pos_first = uniform(a.positions[row0]);
    const int lo_item = (a.window > 0 && pos_first - a.window + 1 > 0) ? pos_first - a.window + 1 : 0;
    const int* bt = a.block_table + static_cast<int64_t>(uniform(a.items[4 * item + 2])) * a.bt_width;

    // this wavefront's tokens and this lane's column
    const int wtok0 = wave * per;
    const int wntok = max(0, min(per, ntok - wtok0));
    const int tc = r / a.gp;
    const int hc = r % a.gp + chunk * 16;
    const bool col_ok = tc < wntok && hc < a.group;
    const int col_row = row0 + (col_ok ? wtok0 + tc : 0);
    const int col_head = g * a.group + (col_ok ? hc : 0);
    const int pos_c = col_ok ? a.positions[col_row] : -1;
    const int lo_c = (a.window > 0 && pos_c - a.window + 1 > 0) ? pos_c - a.window + 1 : 0;
    // keys this wavefront needs at all
    const int whi = uniform(wntok > 0 ? a.positions[row0 + wtok0 + wntok - 1] : -1);
    const int wpos0 = uniform(wntok > 0 ? a.positions[row0 + wtok0] : 0);
    const int wlo = (a.window > 0 && wpos0 - a.window + 1 > 0) ? wpos0 - a.window + 1 : 0;

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

    // The copy of a block: K is 32 rows of D, V is 2 tiles of D rows of 16 keys; both in 16-byte pieces.
    constexpr int K_PIECES = BLOCK_KEYS * D / 8;
    constexpr int V_PIECES = 2 * D * 16 / 8;
    constexpr int K_PER = (K_PIECES + WAVES * PULSE_WAVE - 1) / (WAVES * PULSE_WAVE);
    constexpr int V_PER = (V_PIECES + WAVES * PULSE_WAVE - 1) / (WAVES * PULSE_WAVE);
    u32x4 kreg[K_PER], vreg[V_PER];

    auto fetch = [&](int b) {
        const int j0 = b * BLOCK_KEYS;
        int64_t kbase[2], vbase[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int jt = j0 + 16 * t;
            int pi, slot0;
            page_of(jt, a.page_size, a.page_shift, pi, slot0);
            int page = (jt <= hi && pi < a.bt_width) ? uniform(bt[pi]) : 0;
            page = (page >= 0 && page < a.num_pages) ? page : 0;
            const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
            kbase[t] = (pg * a.page_size + slot0) * D;
            vbase[t] = pg * D * a.page_size + slot0;
        }
#pragma unroll
        for (int i = 0; i < K_PER; ++i) {
            const int piece = tid + i * WAVES * PULSE_WAVE;
            if (piece < K_PIECES) {
                const int key = piece / (D / 8), c8 = piece % (D / 8);
                kreg[i] = *reinterpret_cast<const u32x4*>(a.kc + kbase[key / 16] + static_cast<int64_t>(key % 16) * D + c8 * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < V_PER; ++i) {
            const int piece = tid + i * WAVES * PULSE_WAVE;
            if (piece < V_PIECES) {
                const int t = piece / (D * 2), rest = piece % (D * 2);  // D rows * 2 pieces a row
                const int ch = rest / 2, half = rest % 2;
                vreg[i] = *reinterpret_cast<const u32x4*>(a.vc + vbase[t] + static_cast<int64_t>(ch) * a.page_size + half * 8);
            }
        }
    };
    auto stash = [&](int stage) {
#pragma unroll
        for (int i = 0; i < K_PER; ++i) {
            const int piece = tid + i * WAVES * PULSE_WAVE;
            if (piece < K_PIECES) {
                const int key = piece / (D / 8), c8 = piece % (D / 8);
                *reinterpret_cast<u32x4*>(&s_k[stage][key * KROW + c8 * 8]) = kreg[i];
            }
        }
#pragma unroll
        for (int i = 0; i < V_PER; ++i) {
            const int piece = tid + i * WAVES * PULSE_WAVE;
            if (piece < V_PIECES) {
                const int t = piece / (D * 2), rest = piece % (D * 2);
                const int ch = rest / 2, half = rest % 2;
                const int word = ((t * NDT + ch / 16) * 4 + 2 * half) * VGROUP + ch % 16;  // key groups 2*half, 2*half+1
                *reinterpret_cast<u32x2*>(&s_v[stage][word * 4]) = u32x2{vreg[i][0], vreg[i][1]};
                *reinterpret_cast<u32x2*>(&s_v[stage][(word + VGROUP) * 4]) = u32x2{vreg[i][2], vreg[i][3]};
            }
        }
    };

    // lowest position among this wavefront's columns: blocks wholly at or below it (and above every window's
    // start) need no mask at all
    const int wmin_pos = wpos0;
    const int whi_lo = (a.window > 0 && whi - a.window + 1 > 0) ? whi - a.window + 1 : 0;  // highest window start
    const float c2 = a.scale_log2e;

    auto compute = [&](int b, int stage) {
        const int j0 = b * BLOCK_KEYS;
        f32x4 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ch = 0; ch < NCHUNK; ++ch) {
                const int off = ch * 32 + kg * 8;
                const bf16x8 ak = off < D ? *reinterpret_cast<const bf16x8*>(&s_k[stage][(16 * t + r) * KROW + off]) : zero8();
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak, bq[ch], s[t], 0, 0, 0);
            }
        }
        // the maximum is tracked on the raw scores (the scale is positive); p = exp2((s - m) * scale * log2 e)
        const bool inner = (j0 + BLOCK_KEYS - 1 <= wmin_pos) && (j0 >= whi_lo);
        float p[2][4];
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = s[t][i];
                if (!inner) {
                    const int j = j0 + 16 * t + 4 * kg + i;
                    v = (col_ok && j <= pos_c && j >= lo_c) ? v : -INFINITY;
                }
                p[t][i] = v;
                mx = fmaxf(mx, v);
            }
        if (inner && !col_ok) mx = -INFINITY;
        mx = fmaxf(mx, __shfl_xor(mx, 16, PULSE_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, PULSE_WAVE));
        const float m_new = fmaxf(m, mx);
        const bool dead = m_new == -INFINITY;  // no key of this column so far
        const float alpha = dead ? 1.f : __builtin_amdgcn_exp2f((m - m_new) * c2);
        const float shift = dead ? 0.f : -m_new * c2;
        float psum = 0.f;
        bf16x8 pb;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // exp2(-inf) = 0 for masked scores; a dead column keeps -inf + 0 = -inf as well
                const float e = (inner && !col_ok) ? 0.f : __builtin_amdgcn_exp2f(fmaf(p[t][i], c2, shift));
                psum += e;
                pb[4 * t + i] = (__bf16)e;
            }
        l_part = l_part * alpha + psum;
        m = m_new;
        // stale values under keys outside [lo_item, hi] are cleared (see the split kernel)
        const bool edge = (j0 + BLOCK_KEYS - 1 > hi) || (j0 < lo_item);
        // rescale only when some column's maximum moved
        const bool moved = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
        if (moved) {
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) acc[dt] = acc[dt] * alpha;
        }
        if (edge) {
            uint32_t keep[2][2];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int h2 = 0; h2 < 2; ++h2) {
                    const int j = j0 + 16 * t + 4 * kg + 2 * h2;
                    keep[t][h2] = ((j <= hi && j >= lo_item) ? 0x0000ffffu : 0u) |
                                  ((j + 1 <= hi && j + 1 >= lo_item) ? 0xffff0000u : 0u);
                }
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const u32x2 v0 = *reinterpret_cast<const u32x2*>(&s_v[stage][((dt * 4 + kg) * VGROUP + r) * 4]);
                const u32x2 v1 = *reinterpret_cast<const u32x2*>(&s_v[stage][(((NDT + dt) * 4 + kg) * VGROUP + r) * 4]);
                const u32x4 words = {v0[0] & keep[0][0], v0[1] & keep[0][1], v1[0] & keep[1][0], v1[1] & keep[1][1]};
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, words), pb, acc[dt], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const u32x2 v0 = *reinterpret_cast<const u32x2*>(&s_v[stage][((dt * 4 + kg) * VGROUP + r) * 4]);
                const u32x2 v1 = *reinterpret_cast<const u32x2*>(&s_v[stage][(((NDT + dt) * 4 + kg) * VGROUP + r) * 4]);
                const u32x4 words = {v0[0], v0[1], v1[0], v1[1]};
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, words), pb, acc[dt], 0, 0, 0);
            }
        }
    };

    const int first_block = lo_item / BLOCK_KEYS;
    const int last_block = hi / BLOCK_KEYS;
    fetch(first_block);
    stash(0);
    __syncthreads();
    for (int b = first_block; b <= last_block; ++b) {
        const int stage = (b - first_block) & 1;
        if (b < last_block) fetch(b + 1);
        // a wavefront skips blocks that none of its columns sees (above its diagonal, below its window)
        if (wntok > 0 && b * BLOCK_KEYS <= whi && b * BLOCK_KEYS + BLOCK_KEYS - 1 >= wlo) compute(b, stage);
        if (b < last_block) stash(stage ^ 1);
        __syncthreads();
    }

    l_part += __shfl_xor(l_part, 16, PULSE_WAVE);
    l_part += __shfl_xor(l_part, 32, PULSE_WAVE);
    if (col_ok) {
        const float inv = l_part > 0.f ? 1.0f / l_part : 0.f;
        bf16_t* dst = a.out + static_cast<int64_t>(col_row) * a.o_stride + static_cast<int64_t>(col_head) * D;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            const uint32_t w0 = static_cast<uint32_t>(f32_to_bf16(acc[dt][0] * inv)) |
                                (static_cast<uint32_t>(f32_to_bf16(acc[dt][1] * inv)) << 16);
            const uint32_t w1 = static_cast<uint32_t>(f32_to_bf16(acc[dt][2] * inv)) |
                                (static_cast<uint32_t>(f32_to_bf16(acc[dt][3] * inv)) << 16);
            *reinterpret_cast<u32x2*>(dst + dt * 16 + 4 * kg) = u32x2{w0, w1};
        }
    }
}

#if PULSE_WIDE
// ---------------------------------------------------------------------------------------------------------
// Prompt portions, wide: the same scheme with CT column tiles a wavefront (CT * 16 / G' tokens) and blocks of
// KT * 16 keys, so that every K and V operand read from LDS feeds CT products and the work around a block (the
// addresses, the loop, the barriers) is spread over CT * KT / 2 times as many scores.  The latencies inside a
// block's chain, not the matrix cores, bound this kernel, so the copy must stay out of that chain: K and V go from
// memory straight into LDS (global_load_lds_dwordx4: 16 bytes a lane, lane i to the wavefront's LDS base + 16 i),
// two stages, the next block on its way while this one is computed, with no register in between.
//
// LDS holds 16-byte pieces without padding; which piece a lane fetches is chosen so that the matrix-core operand
// reads are free of bank conflicts:
//   K: piece c of key j (P = D / 8 pieces a key) sits at slot j * P + (c + piece_rot(j)) % P, so that the key rows
//      which eight neighbouring lanes read for one c lie in eight different 16-byte places of an LDS cycle;
//   V: a tile of 16 keys is D channel rows of 32 bytes; the piece (channel ch, half h) sits at slot
//      (ch / 16) * 32 + h * 16 + ch % 16, so the 16 channel rows of one half are 256 contiguous bytes.
// Needs D in {32, 64, 128} (P a power of two, whole 1 KB chunks a tile).
//
// The loads are written in assembly: the compiler knows nothing of them (it would wait for every one before any LDS
// read), so the waits for them are written here too.  Its own vector loads inside the loop (the block table) only
// ever make it wait longer, never shorter: the counter runs in issue order.
// Where piece c of key row j sits inside the row in LDS: at (c + piece_rot(j)) % P.  The eight key rows that eight
// neighbouring lanes read together are j0 .. j0 + 3 and j0 + 8 .. j0 + 11 (j0 a multiple of 4); the rotation sends
// them to eight different 16-byte places of the 128 bytes that LDS serves in a cycle.
__device__ __forceinline__ constexpr int piece_rot(int j, int P) {
    return P >= 8 ? ((j & 3) | (((j >> 3) & 1) << 2)) : (((j >> 1) & 1) | (((j >> 3) & 1) << 1));
}

template <int CT, int KT, int NW>
struct WideShape {
    static constexpr int BK = KT * 16;                    // keys a block
    static constexpr int P = D / 8;                       // 16-byte pieces a key row
    static constexpr int STAGE_K = BK * D;                // bfloat16 elements
    static constexpr int STAGE_V = KT * D * 16;
    static constexpr int STAGE = STAGE_K + STAGE_V;
    static constexpr int TILE_CHUNKS = 16 * P / 64;       // 1 KB chunks (one load of a wavefront) of a key tile; as many of a value tile
    static_assert(KT == NW, "a wavefront copies one key tile and one value tile of every block");
};

// 16 bytes a lane from memory straight into LDS: lane i's piece lands at lds_base + 16 i (a wavefront-wide address).
__device__ __forceinline__ void load_to_lds(const void* from, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds_base), "v"(from) : "memory", "m0");
}

#if PULSE_WIDE_CT > 2
#define PULSE_WIDE_WAVES_PER_EU __attribute__((amdgpu_waves_per_eu(1, 1)))
#else
#define PULSE_WIDE_WAVES_PER_EU PULSE_ATTN_WAVES_PER_EU
#endif
template <int CT, int KT, int NW>
__global__ __launch_bounds__(NW* PULSE_WAVE) PULSE_WIDE_WAVES_PER_EU void attn_prefill_wide_kernel(MfmaArgs a, int per) {
    using Shape = WideShape<CT, KT, NW>;
    constexpr int BK = Shape::BK;
    static_assert(KT % 2 == 0, "the second product takes pairs of key tiles");
    static_assert(D == 32 || D == 64 || D == 128, "whole 1 KB chunks and a power of two of pieces a key");
    constexpr int P = Shape::P;
    __shared__ __attribute__((aligned(1024))) bf16_t s_kv[2 * Shape::STAGE];  // stage: K block, then V block

    // The second half of the kv heads walks the items backwards: a long item (a late portion of a prompt) then
    // shares its compute unit with a short one instead of another long one, and the longest workgroups, which set
    // the kernel's time, run at a lone workgroup's speed.
    const int item = (blockIdx.y * 2 / gridDim.y) & 1 ? gridDim.x - 1 - blockIdx.x : blockIdx.x;
    const int g = blockIdx.y / a.head_chunks;
    const int chunk = blockIdx.y % a.head_chunks;
    const int tid = threadIdx.x;
    const int wave = uniform(tid / PULSE_WAVE);
    const int lane = tid % PULSE_WAVE;
    const int r = lane % 16;
    const int kg = lane / 16;

    const int row0 = uniform(a.items[4 * item]);
    const int ntok = uniform(a.items[4 * item + 1]);         // at most NW * CT * per
    const int hi = uniform(a.positions[row0 + ntok - 1]);    // last key of the workgroup
    // With splits (grid.z; split_size is a multiple of BK, so blocks never straddle two) a workgroup walks the
    // keys of its split only.  An item all of whose keys lie in the first split is finished here as without
    // splits; the others leave unnormalised partial results for attn_prefill_reduce_kernel.
    const bool splits = a.n_splits > 1;
    const int split = splits ? static_cast<int>(blockIdx.z) : 0;
    const int split_begin = splits ? split * a.split_size : 0;
    if (split_begin > hi) return;                            // no key of the item here; the merge does not read this split
    const int split_last = splits ? min(hi, split_begin + a.split_size - 1) : hi;
    const bool direct = !splits || hi < a.split_size;
    const int pos_first = uniform(a.positions[row0]);
    const int lo_item = (a.window > 0 && pos_first - a.window + 1 > 0) ? pos_first - a.window + 1 : 0;
    const int* bt = a.block_table + static_cast<int64_t>(uniform(a.items[4 * item + 2])) * a.bt_width;

    // this wavefront's column tiles and this lane's column in each
    const int tc = r / a.gp;
    const int hc = r % a.gp + chunk * 16;
    bool col_ok[CT];
    int col_row[CT], pos_c[CT], lo_c[CT];
    int t_hi[CT], t_pos0[CT], t_lo[CT], t_hi_lo[CT];  // per tile: last and first position, lowest and highest window start
    bool t_any[CT];
    int col_head = g * a.group;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int wtok0 = (wave * CT + ct) * per;
        const int wntok = max(0, min(per, ntok - wtok0));
        t_any[ct] = wntok > 0;
        col_ok[ct] = tc < wntok && hc < a.group;
        col_row[ct] = row0 + (col_ok[ct] ? wtok0 + tc : 0);
        pos_c[ct] = col_ok[ct] ? a.positions[col_row[ct]] : -1;
        lo_c[ct] = (a.window > 0 && pos_c[ct] - a.window + 1 > 0) ? pos_c[ct] - a.window + 1 : 0;
        t_hi[ct] = uniform(wntok > 0 ? a.positions[row0 + wtok0 + wntok - 1] : -1);
        t_pos0[ct] = uniform(wntok > 0 ? a.positions[row0 + wtok0] : 0);
        t_lo[ct] = (a.window > 0 && t_pos0[ct] - a.window + 1 > 0) ? t_pos0[ct] - a.window + 1 : 0;
        t_hi_lo[ct] = (a.window > 0 && t_hi[ct] - a.window + 1 > 0) ? t_hi[ct] - a.window + 1 : 0;
    }
    if (hc < a.group) col_head += hc;
    // keys this wavefront needs at all: from its first tile's window to its last tile's diagonal
    int w_hi = -1;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) w_hi = max(w_hi, t_hi[ct]);
    const int w_lo = t_lo[0];

    bf16x8 bq[CT][NCHUNK];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const bf16_t* qrow = a.q + static_cast<int64_t>(col_row[ct]) * a.q_stride + static_cast<int64_t>(col_head) * D;
#pragma unroll
        for (int ch = 0; ch < NCHUNK; ++ch) {
            const int off = ch * 32 + kg * 8;
            bq[ct][ch] = (col_ok[ct] && off < D) ? *reinterpret_cast<const bf16x8*>(qrow + off) : zero8();
        }
    }
    f32x4 acc[CT][NDT];
    float m[CT], l_part[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        m[ct] = -INFINITY;
        l_part[ct] = 0.f;
    }

    // The copy of a block: wavefront w brings key tile w and value tile w, in 1 KB chunks (one load each).  What a
    // lane fetches of a chunk does not depend on the block: its offsets are computed once.  Only the page of the
    // wavefront's tile changes from block to block.
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (void __attribute__((address_space(3)))*)(&s_kv[0])));  // the array's address inside LDS
    int k_from[Shape::TILE_CHUNKS], v_from[Shape::TILE_CHUNKS];
#pragma unroll
    for (int i = 0; i < Shape::TILE_CHUNKS; ++i) {
        const int slot = 64 * i + lane;         // within the tile's 16 * P slots
        const int key = slot / P, pos = slot % P;
        const int c8 = (pos - piece_rot(key, P) + P) % P;
        k_from[i] = key * D + c8 * 8;
        const int blk = slot / 32, half = (slot / 16) % 2, chr = slot % 16;
        v_from[i] = (blk * 16 + chr) * a.page_size + half * 8;
    }
    // The page of this wavefront's tile of block b: read from the block table without a branch (an index beyond
    // the table reads its last entry; what it gives is not used) one block ahead of the copy that needs it.
    auto page_ahead = [&](int b) {
        int pi, slot0;
        page_of(b * BK + 16 * wave, a.page_size, a.page_shift, pi, slot0);
        // A scalar load written here, so that it stays where it is, a block ahead of its use, and is waited for
        // with the scalar counter (page_landed) where it is used.  As a vector load it would share the counter of the
        // copies into LDS, and the compiler, which does not see those, would wait for all of them with it: the
        // next block's copy would have to land before this block is computed.
        const int* entry = bt + min(pi, a.bt_width - 1);
        int page;
        asm volatile("s_load_dword %0, %1, 0x0" : "=s"(page) : "s"(entry) : "memory");
        return page;
    };
    // The register a load was asked into holds nothing until the wait: between the two it must not be copied, which
    // the compiler, to whom the load's result looks ready at once, is free to do wherever values meet (the head of a
    // loop, the end of a branch).  So a load and its wait stand in the same straight piece of code, with nothing but
    // the wait touching the variable in between, and only landed values are carried round the loop.
    auto page_landed = [&](int& page) { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(page) : : "memory"); };
    auto pages_landed = [&](int& one, int& two) {
        asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(one), "+s"(two) : : "memory");
    };
    const int64_t page_elems = static_cast<int64_t>(a.nkv) * a.page_size * D;  // of K and of V alike
    const int head_elems = g * a.page_size * D;
    auto fetch = [&](int b, int page_read, int stage) {
        const int jt = b * BK + 16 * wave;
        int pi, slot0;
        page_of(jt, a.page_size, a.page_shift, pi, slot0);
        int page = (jt <= hi && pi < a.bt_width) ? page_read : 0;
        page = (page >= 0 && page < a.num_pages) ? page : 0;
        const int64_t base = page * page_elems + head_elems;
        const bf16_t* kfrom = a.kc + base + slot0 * D;
        const bf16_t* vfrom = a.vc + base + slot0;
        const uint32_t to = lds0 + stage * (Shape::STAGE * 2) + wave * (Shape::TILE_CHUNKS * 1024);
#pragma unroll
        for (int i = 0; i < Shape::TILE_CHUNKS; ++i) load_to_lds(kfrom + k_from[i], to + i * 1024);
#pragma unroll
        for (int i = 0; i < Shape::TILE_CHUNKS; ++i) load_to_lds(vfrom + v_from[i], to + Shape::STAGE_K * 2 + i * 1024);
    };
    // Operand reads.  Row r of score tile t is not key 16 t + r but key 32 (t / 2) + 8 (r / 4) + 4 (t % 2) + r % 4 of
    // the block: the four rows that lane group kg gets back of tiles 2 ks and 2 ks + 1 are then the eight
    // consecutive keys 32 ks + 8 kg .. + 7, whose values for one channel are one 16-byte piece of the value tile,
    // read whole by one lane (eight lanes a cycle read eight neighbouring pieces: no bank is asked twice; as two
    // 8-byte halves of pieces 16 bytes apart every read took two turns).
    int k_at[2][NCHUNK];
#pragma unroll
    for (int par = 0; par < 2; ++par) {
        const int row = 4 * par + 8 * (r / 4) + r % 4;
#pragma unroll
        for (int ch = 0; ch < NCHUNK; ++ch) k_at[par][ch] = (row * P + (4 * ch + kg + piece_rot(row, P)) % P) * 8;
    }
    const int v_at = (kg >> 1) * D * 16 + ((kg & 1) * 16 + r) * 8;

    const float c2 = a.scale_log2e;
    constexpr float LAZY_BITS = 8.f;
    const float lazy = LAZY_BITS / c2;   // in the raw scores' units
    auto compute = [&](int b, int stage) {
        const int j0 = b * BK;
        const bf16_t* s_k = s_kv + stage * Shape::STAGE;
        const bf16_t* s_v = s_k + Shape::STAGE_K;
        // Operand reads run AHEAD steps in front of the products that use them, in an order that is fixed here (the
        // scheduling fences keep the compiler from regrouping them into bursts that are each waited for in full): a
        // read's latency is then covered by the products of the steps before it, not added to them.
        constexpr int AHEAD = 4;
        f32x4 s[CT][KT];
        {
            constexpr int STEPS = KT * NCHUNK;
            auto k_read = [&](int i) {
                const int t = i / NCHUNK, ch = i % NCHUNK;
                return ch * 32 + kg * 8 < D ? *reinterpret_cast<const bf16x8*>(&s_k[32 * (t / 2) * D + k_at[t % 2][ch]]) : zero8();
            };
            bf16x8 ak[STEPS];
#pragma unroll
            for (int i = 0; i < AHEAD && i < STEPS; ++i) ak[i] = k_read(i);
#pragma unroll
            for (int i = 0; i < STEPS; ++i) {
                const int t = i / NCHUNK, ch = i % NCHUNK;
                if (i + AHEAD < STEPS) ak[i + AHEAD] = k_read(i + AHEAD);
#pragma unroll
                for (int ct = 0; ct < CT; ++ct)
                    s[ct][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak[i], bq[ct][ch],
                                                                       ch == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : s[ct][t], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the first value operands are asked for before the weights are computed, the rest as the products go
        constexpr int V_STEPS = (KT / 2) * NDT;
        auto v_read = [&](int i) {
            const int ks = i / NDT, dt = i % NDT;
            return *reinterpret_cast<const u32x4*>(&s_v[(2 * ks) * D * 16 + dt * 256 + v_at]);
        };
        u32x4 vw[V_STEPS];
#pragma unroll
        for (int i = 0; i < AHEAD && i < V_STEPS; ++i) vw[i] = v_read(i);
        __builtin_amdgcn_sched_barrier(0);
        // the maximum is tracked on the raw scores (the scale is positive); p = exp2((s - m) * scale * log2 e)
        bf16x8 pb[CT][KT / 2];
        bool moved = false;
        float alpha[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            // Most blocks lie wholly below a tile's diagonal and inside its window: every column of the tile sees
            // every key, and nothing is masked (columns that stand for no token or head have q = 0 and are never
            // written).  Only a tile whose first token does not see the block's last key, or one of whose windows
            // starts inside the block, takes the mask: score i of tile t belongs to key j0 + 32 (t / 2) + 4 (t % 2) + 8 kg + i,
            // which is seen when 32 (t / 2) + 4 (t % 2) + i lies in
            // [lim_lo, lim_hi] (two compares and a select a score, on a branch that is the same for the wavefront).
            if (j0 + BK - 1 > t_pos0[ct] || j0 < t_hi_lo[ct] || !t_any[ct]) {
                const int lim_hi = col_ok[ct] ? pos_c[ct] - j0 - 8 * kg : -1;
                const int lim_lo = lo_c[ct] - j0 - 8 * kg;
#pragma unroll
                for (int t = 0; t < KT; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        s[ct][t][i] = (32 * (t / 2) + 4 * (t % 2) + i <= lim_hi && 32 * (t / 2) + 4 * (t % 2) + i >= lim_lo)
                                          ? s[ct][t][i] : -INFINITY;
            }
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < KT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[ct][t][i]);
            mx = fmaxf(mx, __shfl_xor(mx, 16, PULSE_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, PULSE_WAVE));
            // The reference point of the exponents follows the maximum only when that has grown by more than
            // 2^LAZY_BITS in the weights' units: until then weights may exceed 1 (by at most that factor, which float32
            // sums and bfloat16 weights hold with the same relative precision), and the accumulators, which are most of
            // a wavefront's registers, are rescaled in few blocks instead of nearly all.  The result is the same
            // quotient of sums.
            const float m_new = mx > m[ct] + lazy ? mx : m[ct];
            const bool dead = m_new == -INFINITY;  // no key of this column so far
            alpha[ct] = dead ? 1.f : __builtin_amdgcn_exp2f((m[ct] - m_new) * c2);
            const float shift = dead ? 0.f : -m_new * c2;
            float psum = 0.f;
#pragma unroll
            for (int t = 0; t < KT; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // exp2(-inf) = 0 for masked scores; a dead column keeps -inf + 0 = -inf as well
                    const float e = __builtin_amdgcn_exp2f(fmaf(s[ct][t][i], c2, shift));
                    psum += e;
                    pb[ct][t / 2][4 * (t % 2) + i] = (__bf16)e;
                }
            l_part[ct] = l_part[ct] * alpha[ct] + psum;
            m[ct] = m_new;
            moved = moved || alpha[ct] != 1.f;
        }
        // rescale only when some column's maximum moved
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) acc[ct][dt] = acc[ct][dt] * alpha[ct];
        }
        // (values under keys outside [lo_item, hi] have been cleared in LDS by clear_stale before this block is computed)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < V_STEPS; ++i) {
            const int ks = i / NDT, dt = i % NDT;
            if (i + AHEAD < V_STEPS) vw[i + AHEAD] = v_read(i + AHEAD);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vw[i]), pb[ct][ks],
                                                                      acc[ct][dt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Stale values under keys that no column of the item may see (beyond its last position, below its window) must
    // not reach the sums, not even as 0 * (inf or nan).  Only the item's last block and the block its window starts
    // in hold such keys, which the whole workgroup knows from the block's number: there the value tiles are cleared
    // in LDS, a 16-byte piece (8 keys of a channel) a thread, before anybody reads them.
    auto clear_stale = [&](int b, int stage) {
        bf16_t* s_v = s_kv + stage * Shape::STAGE + Shape::STAGE_K;
#pragma unroll
        for (int t = 0; t < KT; ++t)
            for (int piece = tid; piece < 2 * D; piece += NW * PULSE_WAVE) {
                const int j = b * BK + 16 * t + 8 * ((piece / 16) % 2);    // the piece's first key
                u32x4 mask;
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    mask[w] = ((j + 2 * w <= hi && j + 2 * w >= lo_item) ? 0x0000ffffu : 0u) |
                              ((j + 2 * w + 1 <= hi && j + 2 * w + 1 >= lo_item) ? 0xffff0000u : 0u);
                u32x4* at = reinterpret_cast<u32x4*>(s_v + t * D * 16 + piece * 8);
                *at = *at & mask;
            }
    };

    const int first_block = max(lo_item, split_begin) / BK;
    const int last_block = split_last / BK;
    // (a split that lies below the item's window has no block to walk: nothing is fetched, its columns stay empty)
    int page_next = 0;   // the page of block b + 1, landed
    if (first_block <= last_block) {
        int page_first = page_ahead(first_block);
        int page_second = page_ahead(first_block + 1);
        pages_landed(page_first, page_second);
        fetch(first_block, page_first, 0);
        page_next = page_second;
    }
    for (int b = first_block; b <= last_block; ++b) {
        const int stage = (b - first_block) & 1;
        // This block's loads were issued a block ago; nothing else is in flight, so the wait does not depend on a
        // count of loads.
        asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
        __syncthreads();  // every wavefront's part of this block has landed
        if (b < last_block)
            fetch(b + 1, page_next, stage ^ 1);  // that stage was read a block ago; the barrier that ended that block released it
        int page_after = page_ahead(b + 2);      // asked for now (past the walk's end it reads an entry nobody uses),
                                                 // waited for at the end of this block, used in the next
        // a wavefront skips blocks that none of its columns sees (above its diagonal, below its window)
        if (b * BK + BK - 1 > hi || b * BK < lo_item) {   // the same for the whole workgroup
            clear_stale(b, stage);
            __syncthreads();
        }
        if (w_hi >= 0 && b * BK <= w_hi && b * BK + BK - 1 >= w_lo) compute(b, stage);
        page_landed(page_after);
        page_next = page_after;
        __syncthreads();  // everybody has read this block
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        float l = l_part[ct];
        l += __shfl_xor(l, 16, PULSE_WAVE);
        l += __shfl_xor(l, 32, PULSE_WAVE);
        if (col_ok[ct] && direct) {
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            bf16_t* dst = a.out + static_cast<int64_t>(col_row[ct]) * a.o_stride + static_cast<int64_t>(col_head) * D;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                const uint32_t w0 = static_cast<uint32_t>(f32_to_bf16(acc[ct][dt][0] * inv)) |
                                    (static_cast<uint32_t>(f32_to_bf16(acc[ct][dt][1] * inv)) << 16);
                const uint32_t w1 = static_cast<uint32_t>(f32_to_bf16(acc[ct][dt][2] * inv)) |
                                    (static_cast<uint32_t>(f32_to_bf16(acc[ct][dt][3] * inv)) << 16);
                *reinterpret_cast<u32x2*>(dst + dt * 16 + 4 * kg) = u32x2{w0, w1};
            }
        } else if (col_ok[ct]) {
            // the split's share of the column: sums as they are, the maximum in the exponent's units
            const int64_t slot = (static_cast<int64_t>(col_row[ct]) * a.nq + col_head) * a.n_splits + split;
            float* dst = a.part_o + slot * D;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(dst + dt * 16 + 4 * kg) = acc[ct][dt];
            if (kg == 0) {
                a.part_ml[2 * slot] = m[ct] == -INFINITY ? -INFINITY : m[ct] * c2;
                a.part_ml[2 * slot + 1] = l;
            }
        }
    }
}

// The merge of the prompt-portion kernel's splits: out[row, head, :] = sum_z w_z o_z / sum_z w_z l_z with
// w_z = exp2(m_z - max m) over the splits that begin at or below the row's position, in the order of the splits.
// A thread takes four channels of one head; rows of items that were finished in the first split are left alone.
constexpr int PR_THREADS = 256;
constexpr int PR_QUADS = D / 4;
constexpr int PR_HEADS = PR_THREADS / PR_QUADS;

__global__ __launch_bounds__(PR_THREADS) void attn_prefill_reduce_kernel(const float* __restrict__ part_o,
                                                                        const float* __restrict__ part_ml,
                                                                        const int* __restrict__ positions,
                                                                        const int* __restrict__ items, int item_tokens,
                                                                        bf16_t* __restrict__ out, int64_t o_stride, int nq,
                                                                        int n_splits, int split_size) {
    const int item = blockIdx.x / item_tokens;
    const int tok = blockIdx.x % item_tokens;
    const int row0 = items[4 * item];
    const int ntok = items[4 * item + 1];
    if (tok >= ntok) return;
    if (positions[row0 + ntok - 1] < split_size) return;   // the item was finished by its only split
    const int64_t row = row0 + tok;
    const int head = blockIdx.y * PR_HEADS + threadIdx.x / PR_QUADS;
    const int quad = threadIdx.x % PR_QUADS;
    if (head >= nq) return;
    const int valid = min(n_splits, positions[row] / split_size + 1);
    const int64_t base = (row * nq + head) * n_splits;
    float mm = -INFINITY;
    for (int z = 0; z < valid; ++z) mm = fmaxf(mm, part_ml[2 * (base + z)]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float ll = 0.f;
    for (int z = 0; z < valid; ++z) {
        const float mz = part_ml[2 * (base + z)];
        const float wz = mz == -INFINITY ? 0.f : exp2f(mz - mm);
        ll += wz * part_ml[2 * (base + z) + 1];
        // a split below the row's window holds sums of nothing (zeros), never stale memory: it was written
        acc += *reinterpret_cast<const f32x4*>(part_o + (base + z) * D + 4 * quad) * wz;
    }
    const float inv = ll > 0.f ? 1.0f / ll : 0.f;
    const uint32_t w0 = static_cast<uint32_t>(f32_to_bf16(acc[0] * inv)) | (static_cast<uint32_t>(f32_to_bf16(acc[1] * inv)) << 16);
    const uint32_t w1 = static_cast<uint32_t>(f32_to_bf16(acc[2] * inv)) | (static_cast<uint32_t>(f32_to_bf16(acc[3] * inv)) << 16);
    *reinterpret_cast<u32x2*>(out + row * o_stride + static_cast<int64_t>(head) * D + 4 * quad) = u32x2{w0, w1};
}

#endif  // PULSE_WIDE

// out[row, head, :] = sum_z w_z o_z / sum_z w_z l_z with w_z = exp2(m_z - max m), over the splits that hold keys of
// the row.  One workgroup per (row, `hpw` heads): its groups of threads are dealt out over the heads, a head's groups
// over the splits (with few splits a workgroup would otherwise be mostly idle, and the launch eight times as wide).
// The splits' (m, l) pairs go through LDS, and the partial outputs of the first splits are asked for before anything
// waits, so that the kernel is little more than two trips to memory.
constexpr int MAX_SPLITS = 1024;

constexpr int REDUCE_THREADS = 256;
constexpr int REDUCE_QUADS = D / 4;                              // float4 pieces of a head
constexpr int REDUCE_GROUPS = REDUCE_THREADS / REDUCE_QUADS;     // groups of threads that share heads and splits out

__global__ __launch_bounds__(REDUCE_THREADS) void attn_mfma_reduce_kernel(const float* __restrict__ part_o,
                                                                         const float* __restrict__ part_ml,
                                                                         const int* __restrict__ positions,
                                                                         const int* __restrict__ items, int per,
                                                                         bf16_t* __restrict__ out, int64_t o_stride, int nq,
                                                                         int n_splits, int static_split_size, int hpw_log2,
                                                                         const int* __restrict__ live_context,
                                                                         const int* __restrict__ plan, int n_items) {
    __shared__ float s_w[MAX_SPLITS];      // hpw * n_splits <= MAX_SPLITS (hpw > 1 only with few splits)
    __shared__ float s_l[MAX_SPLITS];
    __shared__ f32x4 s_acc[REDUCE_GROUPS][REDUCE_QUADS];
    // The kernel is a chain of trips to memory and little else, so it is kept to two: the item (and what says how its
    // keys were cut), then everything that needs only the row: its position, the item's last position, the (m, l)
    // pairs of every split and the first partial outputs.  What of that a row does not use is read and dropped.
    const int item = blockIdx.x / per;
    const int tok = blockIdx.x % per;
    const int row0 = items ? items[4 * item] : item, ntok = items ? items[4 * item + 1] : 1;   // (null: item i is token i)
    const int split_size = plan ? plan[1 + n_items * n_splits + item]
                           : live_context ? live_split_size(*live_context, n_splits, static_split_size) : static_split_size;
    if (tok >= ntok) return;   // only the rows of this launch's items have partial results
    const int64_t row = row0 + tok;
    const int hpw = 1 << hpw_log2;            // heads of this workgroup
    const int head0 = blockIdx.y * hpw;
    const int pos_row = positions[row];
    const int pos_last = positions[row0 + ntok - 1];
    constexpr int ML_PER = MAX_SPLITS / REDUCE_THREADS;
    f32x2 ml[ML_PER];
#pragma unroll
    for (int j = 0; j < ML_PER; ++j) {
        const int i = threadIdx.x + j * REDUCE_THREADS;
        const int hs = i & (hpw - 1), z = i >> hpw_log2;
        ml[j] = f32x2{0.f, 0.f};
        if (i < hpw * n_splits && head0 + hs < nq)
            ml[j] = *reinterpret_cast<const f32x2*>(part_ml + 2 * ((row * nq + head0 + hs) * n_splits + z));
    }
    // group `grp` of threads takes head grp % hpw and of its splits sg = grp / hpw, sg + gph, ..; a thread four
    // channels of them.
    // The partial outputs are asked for before the weights are known, eight splits of a group at a time.
    const int gph = REDUCE_GROUPS >> hpw_log2;   // groups a head
    const int quad = threadIdx.x % REDUCE_QUADS;
    const int grp = threadIdx.x / REDUCE_QUADS;
    const int hs = grp & (hpw - 1);
    const int sg = grp >> hpw_log2;
    const int head = head0 + hs;
    const bool works = sg < gph && head < nq;
    const int64_t base = (row * nq + (works ? head : head0)) * n_splits;
    const float* my_w = s_w + (works ? hs : 0) * n_splits;
    const float* my_l = s_l + (works ? hs : 0) * n_splits;
    constexpr int AHEAD = 8;
    f32x4 first[AHEAD];
#pragma unroll
    for (int i = 0; i < AHEAD; ++i) {
        const int z = sg + i * gph;
        // a split without keys of the row left nothing behind: what is read there is not used (z < valid below)
        first[i] = (works && z < n_splits) ? *reinterpret_cast<const f32x4*>(part_o + (base + z) * D + 4 * quad)
                                           : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (plan && pos_last < split_size) return;   // the item was finished by its only split
    const int valid = min(n_splits, pos_row / split_size + 1);
#pragma unroll
    for (int j = 0; j < ML_PER; ++j) {
        const int i = threadIdx.x + j * REDUCE_THREADS;
        const int hs2 = i & (hpw - 1), z = i >> hpw_log2;
        if (i < hpw * valid && head0 + hs2 < nq) {
            s_w[hs2 * n_splits + z] = ml[j][0];
            s_l[hs2 * n_splits + z] = ml[j][1];
        }
    }
    __syncthreads();
    float inv = 0.f;
    if (works) {
        float mm = -INFINITY;
        for (int z = 0; z < valid; ++z) mm = fmaxf(mm, my_w[z]);
        float ll = 0.f;
        for (int z = 0; z < valid; ++z) ll += (my_w[z] == -INFINITY ? 0.f : exp2f(my_w[z] - mm)) * my_l[z];
        inv = ll > 0.f ? 1.0f / ll : 0.f;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) {
            const int z = sg + i * gph;
            if (z < valid) acc += first[i] * (my_w[z] == -INFINITY ? 0.f : exp2f(my_w[z] - mm));
        }
        for (int z = sg + AHEAD * gph; z < valid; z += gph) {
            const float wz = my_w[z] == -INFINITY ? 0.f : exp2f(my_w[z] - mm);
            acc += *reinterpret_cast<const f32x4*>(part_o + (base + z) * D + 4 * quad) * wz;
        }
        s_acc[grp][quad] = acc;
    }
    __syncthreads();
    // a head's groups' sums in a fixed order
    if (works && sg == 0) {
        f32x4 v = s_acc[grp][quad];
        for (int gi = 1; gi < gph; ++gi) v += s_acc[grp + gi * hpw][quad];
        bf16_t* dst = out + row * o_stride + static_cast<int64_t>(head) * D + 4 * quad;
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[e] = f32_to_bf16(v[e] * inv);
    }
}

// The plan of a step of decoded tokens and short portions whose contexts differ much: how many splits every item's
// keys are cut into, and in which order the workgroups take the (item, split) pairs.  The smallest split length T
// (whole 32-key blocks, at least min_keys) with sum_i min(n_splits, ceil(context_i / T)) <= slots is found; item i
// is cut evenly into that many splits; the pairs are ordered by their lengths, longest first, the second
// `first_wave` of them the other way round: consecutive workgroups go to different compute units until every unit
// has one, so the longest walks start first, each on a unit of its own, and the unit that got the longest gets the
// shortest of the second round.  One workgroup; n_items * n_splits <= PLAN_MAX_PAIRS.
constexpr int PLAN_THREADS = 256;
constexpr int PLAN_MAX_PAIRS = 1024;

__global__ __launch_bounds__(PLAN_THREADS) void attn_plan_kernel(const int* __restrict__ items,
                                                                  const int* __restrict__ positions, int n_items,
                                                                  int n_splits, int slots, int first_wave, int min_keys,
                                                                  int* __restrict__ plan) {
    __shared__ int s_ctx[PLAN_MAX_PAIRS];
    __shared__ int s_size[PLAN_MAX_PAIRS];
    __shared__ int s_len[PLAN_MAX_PAIRS];
    __shared__ int s_pair[PLAN_MAX_PAIRS];
    __shared__ int s_red[PLAN_THREADS / PULSE_WAVE];
    const int tid = threadIdx.x, lane = tid % PULSE_WAVE, wave = tid / PULSE_WAVE;
    constexpr int WV = PLAN_THREADS / PULSE_WAVE;
    // a sum or a maximum over the workgroup, the same in every thread
    auto all_sum = [&](int v) {
#pragma unroll
        for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PULSE_WAVE);
        __syncthreads();   // (the last round's reads of s_red are over)
        if (lane == 0) s_red[wave] = v;
        __syncthreads();
        int t = 0;
#pragma unroll
        for (int w = 0; w < WV; ++w) t += s_red[w];
        return t;
    };
    int longest = 1;
    for (int i = tid; i < n_items; i += PLAN_THREADS) {
        const int c = positions[items ? items[4 * i] + items[4 * i + 1] - 1 : i] + 1;
        s_ctx[i] = c;
        longest = max(longest, c);
    }
#pragma unroll
    for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) longest = max(longest, __shfl_xor(longest, off, PULSE_WAVE));
    if (lane == 0) s_red[wave] = longest;
    __syncthreads();
    longest = 0;
#pragma unroll
    for (int w = 0; w < WV; ++w) longest = max(longest, s_red[w]);
    // T in blocks of 32 keys: the smallest in [lo, hi] whose pairs fit the slots (hi: every item whole)
    int lo = max(1, (min_keys + 31) / 32), hi = (longest + 31) / 32;
    lo = min(lo, hi);
    while (lo < hi) {
        const int mid = (lo + hi) / 2, t = mid * 32;
        int mine = 0;
        for (int i = tid; i < n_items; i += PLAN_THREADS) mine += min(n_splits, (s_ctx[i] + t - 1) / t);
        if (all_sum(mine) <= slots) hi = mid; else lo = mid + 1;
    }
    const int T = lo * 32;
    // every item's split size and number of pairs; the pairs' places by a running sum over the items
    constexpr int PER = PLAN_MAX_PAIRS / PLAN_THREADS;   // consecutive items a thread
    int counts[PER], run = 0;
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const int i = tid * PER + e;
        counts[e] = 0;
        if (i < n_items) {
            const int c = s_ctx[i];
            const int n = min(n_splits, (c + T - 1) / T);
            const int size = ((c + n - 1) / n + 31) / 32 * 32;
            s_size[i] = size;
            plan[1 + n_items * n_splits + i] = size;
            counts[e] = (c + size - 1) / size;
        }
        run += counts[e];
    }
    int incl = run;   // inclusive sum over the threads before: within the wavefront, then over the wavefronts
#pragma unroll
    for (int off = 1; off < PULSE_WAVE; off <<= 1) {
        const int up = __shfl_up(incl, off, PULSE_WAVE);
        if (lane >= off) incl += up;
    }
    __syncthreads();
    if (lane == PULSE_WAVE - 1) s_red[wave] = incl;
    __syncthreads();
    int before = incl - run, total = 0;
#pragma unroll
    for (int w = 0; w < WV; ++w) {
        if (w < wave) before += s_red[w];
        total += s_red[w];
    }
#pragma unroll
    for (int e = 0; e < PER; ++e) {
        const int i = tid * PER + e;
        if (i < n_items) {
            const int c = s_ctx[i], size = s_size[i];
            for (int z = 0; z < counts[e]; ++z) {
                s_len[before + z] = min(size, c - z * size);
                s_pair[before + z] = i * n_splits + z;
            }
            before += counts[e];
        }
    }
    __syncthreads();
    // a pair's place: how many are longer (or as long and earlier); the second round turned round
    const int second_end = min(2 * first_wave, total);
    for (int j = tid; j < total; j += PLAN_THREADS) {
        const int mine = s_len[j];
        int rank = 0;
        for (int k = 0; k < total; ++k) rank += (s_len[k] > mine || (s_len[k] == mine && k < j)) ? 1 : 0;
        const int place = (rank >= first_wave && rank < second_end) ? first_wave + (second_end - 1 - rank) : rank;
        plan[1 + place] = s_pair[j];
    }
    if (tid == 0) plan[0] = total;
}

}  // namespace

extern "C" int pulse_attn_mfma_head_dim() { return D; }

namespace {

struct Preparation {
    const void* q_w;
    const void* k_w;
    const float* cos_t;
    const float* sin_t;
    float eps;
    int rotary_dim, pairing, new_key;
};

int launch_attn_mfma(const void* q, int64_t q_stride, void* out, int64_t o_stride, const void* kcache,
                     const void* vcache, const int* positions, const int* block_table, int bt_width, const int* items,
                     int n_items, int tokens, int nq, int nkv, int page_size, int num_pages, float scale, int window,
                     int split_size, int n_splits, int max_context, float* part_o, float* part_ml,
                     const Preparation* prep, const int* live_context, const int* plan, hipStream_t stream) {
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
    PULSE_REQUIRE(n_splits == 1 || (part_o && part_ml && (reinterpret_cast<uintptr_t>(part_o) % 16) == 0),
                  "attn_mfma: scratch is missing or not 16-byte aligned");
    PULSE_REQUIRE(n_splits <= MAX_SPLITS, "attn_mfma: at most %d splits, got %d", MAX_SPLITS, n_splits);
    PULSE_REQUIRE(n_splits < 65536 && static_cast<int64_t>(n_items) * nkv * ((nq / nkv + 15) / 16) * n_splits < (int64_t{1} << 31), "attn_mfma: grid too large");
    PULSE_REQUIRE(q && out && kcache && vcache && positions && block_table, "attn_mfma: null pointer");
    PULSE_REQUIRE(items || (prep && n_items == tokens), "attn_mfma: only decoded tokens, one an item, can do without a list of items");
    if (tokens == 0 || n_items == 0) return 0;
    const int group = nq / nkv;
    int gp = 1;
    while (gp < group && gp < 16) gp *= 2;
    MfmaArgs a;
    a.q = static_cast<const bf16_t*>(q); a.q_stride = q_stride;
    a.out = static_cast<bf16_t*>(out); a.o_stride = o_stride;
    a.part_o = part_o; a.part_ml = part_ml;
    a.kc = static_cast<const bf16_t*>(kcache); a.vc = static_cast<const bf16_t*>(vcache);
    a.positions = positions; a.block_table = block_table; a.items = items;
    a.bt_width = bt_width; a.nq = nq; a.nkv = nkv; a.group = group; a.gp = gp; a.head_chunks = (group + 15) / 16;
    a.page_size = page_size; a.num_pages = num_pages;
    a.page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
    a.scale_log2e = scale * 1.4426950408889634f;
    a.window = window; a.split_size = split_size; a.n_splits = n_splits;
    a.live_context = n_splits > 1 ? live_context : nullptr;
    a.plan = n_splits > 1 ? plan : nullptr;
    a.n_items = n_items;
    a.q_w = a.k_w = nullptr; a.cos_t = a.sin_t = nullptr; a.eps = 0.f; a.rotary_dim = 0; a.pairing = 0; a.new_key = 0;
    if (prep) {
        a.q_w = static_cast<const bf16_t*>(prep->q_w); a.k_w = static_cast<const bf16_t*>(prep->k_w);
        a.cos_t = prep->cos_t; a.sin_t = prep->sin_t; a.eps = prep->eps; a.rotary_dim = prep->rotary_dim;
        a.pairing = prep->pairing; a.new_key = prep->new_key;
        hipLaunchKernelGGL(attn_mfma_kernel<true>, dim3(n_items * nkv * a.head_chunks * n_splits), dim3(WAVES * PULSE_WAVE),
                           0, stream, a);
    } else {
        hipLaunchKernelGGL(attn_mfma_kernel<false>, dim3(n_items * nkv * a.head_chunks * n_splits), dim3(WAVES * PULSE_WAVE),
                           0, stream, a);
    }
    PULSE_LAUNCH_CHECK("attn_mfma");
    if (n_splits > 1) {
        const int per = prep ? 1 : 16 / gp;   // tokens an item may hold: decoded tokens come one an item
        int hpw = 1, hpw_log2 = 0;            // heads a workgroup: as many as leave every split of a head a group of threads
        while (hpw * 2 * n_splits <= REDUCE_GROUPS && hpw * 2 <= nq) { hpw *= 2; ++hpw_log2; }
        hipLaunchKernelGGL(attn_mfma_reduce_kernel, dim3(n_items * per, (nq + hpw - 1) / hpw), dim3(REDUCE_THREADS), 0, stream,
                           part_o, part_ml, positions, items, per, a.out, o_stride, nq, n_splits, split_size, hpw_log2,
                           a.live_context, a.plan, n_items);
        PULSE_LAUNCH_CHECK("attn_mfma_reduce");
    }
    return 0;
}

}  // namespace

// Scratch needed for `tokens` rows cut into `n_splits`: tokens * nq * n_splits * D floats of part_o, * 2 of part_ml.
// live_context (device, or null): the longest context (last position + 1) among ALL items of this call as the step
// has it; split_size and n_splits say what the launch is made for (max_context), and with live_context the kernel cuts
// the keys that are there evenly into the same number of splits.  A value below an item's context loses keys.
// plan (device, or null): what pulse_attn_plan made of these items and positions for this n_splits; it takes the
// place of that even cut (every item then has a split size of its own and the workgroups an order).
extern "C" int pulse_attn_mfma(const void* q, int64_t q_stride, void* out, int64_t o_stride, const void* kcache,
                               const void* vcache, const int* positions, const int* block_table, int bt_width,
                               const int* items, int n_items, int tokens, int nq,
                               int nkv, int page_size, int num_pages, float scale, int window, int split_size,
                               int n_splits, int max_context, float* part_o, float* part_ml, const int* live_context,
                               const int* plan, hipStream_t stream) {
    return launch_attn_mfma(q, q_stride, out, o_stride, kcache, vcache, positions, block_table, bt_width, items, n_items,
                            tokens, nq, nkv, page_size, num_pages, scale, window, split_size, n_splits, max_context,
                            part_o, part_ml, nullptr, live_context, plan, stream);
}

// The plan of a step (see attn_plan_kernel) for pulse_attn_mfma / pulse_attn_decode with the same items and n_splits:
// plan holds 1 + n_items * n_splits + n_items ints.  slots: how many workgroups a kv head's walks should be cut into
// at most (what the compute units hold at a time); first_wave: how many of them land on units of their own.
extern "C" int pulse_attn_plan_max_pairs() { return PLAN_MAX_PAIRS; }

extern "C" int pulse_attn_plan(const int* items, const int* positions, int n_items, int n_splits, int slots,
                               int first_wave, int min_keys, int* plan, hipStream_t stream) {
    PULSE_REQUIRE(positions && plan, "attn_plan: null pointer");   // (items may be null: item i is token i)
    PULSE_REQUIRE(n_items >= 1 && n_splits >= 1 && static_cast<int64_t>(n_items) * n_splits <= PLAN_MAX_PAIRS,
                  "attn_plan: %d items in up to %d splits are more than %d pairs", n_items, n_splits, PLAN_MAX_PAIRS);
    PULSE_REQUIRE(slots >= 1 && first_wave >= 1 && min_keys >= 1, "attn_plan: slots, first_wave and min_keys must be positive");
    hipLaunchKernelGGL(attn_plan_kernel, dim3(1), dim3(PLAN_THREADS), 0, stream, items, positions, n_items, n_splits,
                       slots, first_wave, min_keys, plan);
    PULSE_LAUNCH_CHECK("attn_plan");
    return 0;
}

// Whether pulse_attn_decode takes a rotation: whole 8-element slices, and for pairs (i, i + rotary_dim / 2) a
// partner slice in the same lane.
extern "C" int pulse_attn_decode_takes(int rotary_dim, int pairing) {
    if (rotary_dim == 0) return 1;
    if (rotary_dim < 0 || rotary_dim > D || rotary_dim % 8) return 0;
    return pairing == 0 || (pairing == 1 && rotary_dim % 64 == 0);
}

// Attention for decoded tokens straight from the raw projection output: every item holds ONE token; qkv is
// [tokens, (nq + 2 nkv) D] bfloat16 (q heads, k heads, v heads; row stride qkv_stride).  Per-head RMSNorm (q_w, k_w
// bfloat16 [D], or null) and rotation (cos_t, sin_t float32 [tokens, rotary_dim / 2], or null) of q and, with new_key,
// of the token's key happen inside; with new_key the key and the value are also written to the token's page (kcache
// and vcache are written then).  Without new_key the pages already hold the token (a run that reads another run's
// cache).  items may be null: item i is then token i with row i of the block table.  The rest as pulse_attn_mfma.
extern "C" int pulse_attn_decode(const void* qkv, int64_t qkv_stride, void* out, int64_t o_stride, void* kcache,
                                 void* vcache, const int* positions, const int* block_table, int bt_width,
                                 const int* items, int n_items, int tokens, int nq, int nkv, int page_size,
                                 int num_pages, float scale, int window, int split_size, int n_splits, int max_context,
                                 float* part_o, float* part_ml, const void* q_w, const void* k_w, float eps,
                                 const float* cos_t, const float* sin_t, int rotary_dim, int pairing, int new_key,
                                 const int* live_context, const int* plan, hipStream_t stream) {
    PULSE_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attn_decode: cos and sin come together");
    if (!cos_t) rotary_dim = 0;
    PULSE_REQUIRE(pulse_attn_decode_takes(rotary_dim, pairing), "attn_decode: rotation of %d channels with pairing %d is not "
                  "supported for head size %d", rotary_dim, pairing, D);
    PULSE_REQUIRE((reinterpret_cast<uintptr_t>(q_w) % 16) == 0 && (reinterpret_cast<uintptr_t>(k_w) % 16) == 0 &&
                  (reinterpret_cast<uintptr_t>(cos_t) % 16) == 0 && (reinterpret_cast<uintptr_t>(sin_t) % 16) == 0,
                  "attn_decode: norm weights and rotation tables must be 16-byte aligned");
    PULSE_REQUIRE(nq > 0 && nkv > 0 && qkv_stride >= static_cast<int64_t>(nq + (new_key ? 2 * nkv : 0)) * D,
                  "attn_decode: the projection output's rows are too short");
    PULSE_REQUIRE(n_items == tokens, "attn_decode: %d items for %d tokens (every item holds one token)", n_items, tokens);
    Preparation prep{q_w, k_w, cos_t, sin_t, eps, rotary_dim, pairing, new_key ? 1 : 0};
    return launch_attn_mfma(qkv, qkv_stride, out, o_stride, kcache, vcache, positions, block_table, bt_width, items,
                            n_items, tokens, nq, nkv, page_size, num_pages, scale, window, split_size, n_splits,
                            max_context, part_o, part_ml, &prep, live_context, plan, stream);
}

// Keys a split of the prompt-portion kernel must be a multiple of; 0 when this head size's kernel has no splits.
extern "C" int pulse_attn_prefill_split_keys() { return PULSE_WIDE ? 64 : 0; }

// Prompt portions: items of up to 4 * pulse_attn_prefill_tiles() * pulse_attn_mfma_tokens_per_item(group) tokens of one
// request, a workgroup each (and per split), keys shared through LDS.  With n_splits > 1 (head sizes for which
// pulse_attn_prefill_split_keys() > 0) the keys are cut into splits of split_size keys; part_o holds
// tokens * nq * n_splits * D floats and part_ml tokens * nq * n_splits * 2, as for pulse_attn_mfma.
extern "C" int pulse_attn_prefill(const void* q, int64_t q_stride, void* out, int64_t o_stride, const void* kcache,
                                  const void* vcache, const int* positions, const int* block_table, int bt_width,
                                  const int* items, int n_items, int tokens,
                                  int nq, int nkv, int page_size, int num_pages, float scale, int window,
                                  int split_size, int n_splits, float* part_o, float* part_ml, hipStream_t stream) {
    PULSE_REQUIRE(n_splits >= 1 && n_splits < 65536, "attn_prefill: bad number of splits %d", n_splits);
    if (n_splits > 1) {
        PULSE_REQUIRE(pulse_attn_prefill_split_keys() > 0, "attn_prefill: head size %d has no split variant", D);
        PULSE_REQUIRE(split_size > 0 && split_size % pulse_attn_prefill_split_keys() == 0,
                      "attn_prefill: split size %d must be a positive multiple of %d", split_size, pulse_attn_prefill_split_keys());
        PULSE_REQUIRE(part_o && part_ml && (reinterpret_cast<uintptr_t>(part_o) % 16) == 0,
                      "attn_prefill: scratch for the split results is missing or not 16-byte aligned");
    }
    PULSE_REQUIRE(tokens >= 0 && n_items >= 0 && nq > 0 && nkv > 0, "attn_prefill: bad sizes");
    PULSE_REQUIRE(nq % nkv == 0, "attn_prefill: %d query heads are not a multiple of %d kv heads", nq, nkv);
    PULSE_REQUIRE(page_size > 0 && page_size % 16 == 0, "attn_prefill: page size %d must be a multiple of 16", page_size);
    PULSE_REQUIRE(num_pages > 0 && bt_width > 0 && window >= 0, "attn_prefill: bad cache geometry");
    PULSE_REQUIRE(q_stride % 8 == 0 && o_stride % 4 == 0 && q_stride >= static_cast<int64_t>(nq) * D &&
                  o_stride >= static_cast<int64_t>(nq) * D, "attn_prefill: row strides must cover the heads and keep alignment");
    PULSE_REQUIRE((reinterpret_cast<uintptr_t>(q) % 16) == 0 && (reinterpret_cast<uintptr_t>(kcache) % 16) == 0 &&
                  (reinterpret_cast<uintptr_t>(vcache) % 16) == 0 && (reinterpret_cast<uintptr_t>(out) % 8) == 0,
                  "attn_prefill: pointers must be 16-byte aligned");
    PULSE_REQUIRE(static_cast<int64_t>(nkv) * ((nq / nkv + 15) / 16) < 65536, "attn_prefill: grid too large");
    PULSE_REQUIRE(q && out && kcache && vcache && positions && block_table && items, "attn_prefill: null pointer");
    if (tokens == 0 || n_items == 0) return 0;
    const int group = nq / nkv;
    int gp = 1;
    while (gp < group && gp < 16) gp *= 2;
    MfmaArgs a;
    a.q = static_cast<const bf16_t*>(q); a.q_stride = q_stride;
    a.out = static_cast<bf16_t*>(out); a.o_stride = o_stride;
    a.part_o = nullptr; a.part_ml = nullptr;
    a.kc = static_cast<const bf16_t*>(kcache); a.vc = static_cast<const bf16_t*>(vcache);
    a.positions = positions; a.block_table = block_table; a.items = items;
    a.bt_width = bt_width; a.nq = nq; a.nkv = nkv; a.group = group; a.gp = gp; a.head_chunks = (group + 15) / 16;
    a.page_size = page_size; a.num_pages = num_pages;
    a.page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
    a.scale_log2e = scale * 1.4426950408889634f;
    a.window = window; a.split_size = n_splits > 1 ? split_size : 0; a.n_splits = n_splits;
    a.live_context = nullptr;
    a.plan = nullptr;
    a.part_o = n_splits > 1 ? part_o : nullptr; a.part_ml = n_splits > 1 ? part_ml : nullptr;
#if PULSE_WIDE
    hipLaunchKernelGGL((attn_prefill_wide_kernel<WIDE_CT, 4, WIDE_NW>), dim3(n_items, nkv * a.head_chunks, n_splits),
                       dim3(WIDE_NW * PULSE_WAVE), 0, stream, a, 16 / gp);
    if (n_splits > 1) {
        PULSE_LAUNCH_CHECK("attn_prefill");
        const int item_tokens = WIDE_NW * WIDE_CT * (16 / gp);
        hipLaunchKernelGGL(attn_prefill_reduce_kernel, dim3(n_items * item_tokens, (nq + PR_HEADS - 1) / PR_HEADS),
                           dim3(PR_THREADS), 0, stream, part_o, part_ml, positions, items, item_tokens, a.out, o_stride, nq,
                           n_splits, split_size);
    }
#else
    hipLaunchKernelGGL(attn_prefill_kernel, dim3(n_items, nkv * a.head_chunks), dim3(WAVES * PULSE_WAVE), 0, stream, a,
                       16 / gp);
#endif
    PULSE_LAUNCH_CHECK("attn_prefill");
    return 0;
}

// Column tiles a wavefront of the prompt-portion kernel takes: its items hold 4 * this * tokens_per_item tokens.
extern "C" int pulse_attn_prefill_tiles() { return PREFILL_TILES; }

// Columns per token and tokens per item for a group size: the host builds its item list with these.
extern "C" int pulse_attn_mfma_tokens_per_item(int group) {
    int gp = 1;
    while (gp < group && gp < 16) gp *= 2;
    return 16 / gp;
}
