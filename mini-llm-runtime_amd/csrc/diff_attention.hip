// Differential attention over the paged cache.
//
// A query head holds two maps: two softmax attentions with queries and keys of their own (head_dim channels
// each, laid out [map 1 | map 2] within a head) over the SAME values (value_dim channels).  The head's output
// is o = a1 - lam * a2, divided by its root mean square over the value channels (eps inside the root), times
// out_scale, times an activation of the head's gate.  Scores: (q . k) * scale * temp(p), the query's factor
// temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1) growing with its position p; then, with a cap,
// score <- cap * tanh(score / cap); position p sees the keys 0 .. p, or with a mask rule only the last `mask_size`
// of them (window) or those of its own block of `mask_size` positions counted from 0 (chunk).  All of this is
// 32-bit.  Queries and keys may be rotated on their way (`diff_qkv_prep_kernel`): the first `rot` channels of each
// map of each head, in pairs (j, j + rot / 2) or (2 j, 2 j + 1), by the angles of the position's table row.
//
// Cache of one layer: keys pages[num_pages][kv_heads][page_size][2 * head_dim]; values transposed within a
// page, pages[num_pages][kv_heads][value_dim][page_size], so that the keys of one channel lie side by side (the
// operand layout of the matrix cores for probabilities x values).  Query head h reads kv head
// h / (q_heads / kv_heads).
//
// `diff_attention_partial_kernel`: one wavefront per (token, head and map, key range).  Key ranges are
// [s * split_keys, (s + 1) * split_keys) in absolute positions and tiles of 64 keys start at multiples of 64, so
// the order of a token's sums follows from its own position alone, never from the batch around it or from how
// its request was cut into steps.  It leaves (max, sum, weighted values) per range;
// `diff_attention_combine_kernel` merges the ranges in ascending order, takes the difference of the maps, norms
// and gates.  Both serve the float engine for every token, and the bfloat16 engine for single tokens and short
// portions (and for the sizes that the matrix-core kernel does not take).
//
// `diff_attention_tiles_kernel` (bfloat16): prompt portions on the matrix cores.  A workgroup takes up to 64
// consecutive tokens of one request and up to four query heads of one kv head; a wavefront 16 tokens of one head,
// both maps.  Keys and values are staged once per workgroup through LDS in tiles of 32 keys and serve both maps of
// all its heads; the head's epilogue (difference, norm, gate) runs in registers.
#include "common.h"

#define TILE_KEYS 64
#define DIM_CHUNK 64
#define MAX_V_REGS 4            // value_dim <= 64 * MAX_V_REGS
#define COMBINE_MAX_SPLITS 1024

struct DiffArgs {
    const elem_t* q; long q_stride;            // q[m * q_stride + (head * 2 + map) * head_dim + d]
    const elem_t* k_pages; const elem_t* v_pages;
    const int32_t* block_table; const int32_t* slots; const int32_t* positions;
    const elem_t* gate; long gate_stride;      // gate[m * gate_stride + head * value_dim + c], or null
    elem_t* out;                               // [rows, q_heads * value_dim]
    float* partial;                            // [rows, q_heads * 2, max_splits, value_dim + 2]
    int max_blocks, q_heads, kv_heads, head_dim, value_dim, page_size, split_keys, max_splits;
    float scale, softcap, temp_coef, temp_every, lam, out_scale, eps;
    // which rows: null: blockIdx.x is the batch row; else blockIdx.x = group * group_tokens + i stands for row
    // group_first[group] + i while i < group_count[group] (partial results are indexed by blockIdx.x)
    const int32_t* group_first; const int32_t* group_count; int group_tokens;
    int mask_kind, mask_size;                  // 0: every earlier key; 1: the last mask_size positions; 2: the query's block
};

#define MASK_NONE 0
#define MASK_WINDOW 1
#define MASK_CHUNK 2
// The first key that a query at `pos` sees (never decreasing in pos).
__device__ __forceinline__ int first_key(const DiffArgs& a, int pos) {
    if (a.mask_kind == MASK_WINDOW) return max(0, pos - a.mask_size + 1);
    if (a.mask_kind == MASK_CHUNK) return (pos / a.mask_size) * a.mask_size;
    return 0;
}

__device__ __forceinline__ int diff_row(const DiffArgs& a) {
    if (a.group_first == nullptr) return blockIdx.x;
    const int g = blockIdx.x / a.group_tokens, i = blockIdx.x % a.group_tokens;
    return i < a.group_count[g] ? a.group_first[g] + i : -1;
}

// Writes the step's keys [kv_heads][2 * head_dim] and values [kv_heads][value_dim] into their pages.
__global__ void diff_kv_write_kernel(const elem_t* __restrict__ k, long k_stride, const elem_t* __restrict__ v, long v_stride,
                                     elem_t* __restrict__ k_pages, elem_t* __restrict__ v_pages,
                                     const int32_t* __restrict__ block_table, int max_blocks,
                                     const int32_t* __restrict__ slots, const int32_t* __restrict__ positions, int kv_heads,
                                     int key_dim, int value_dim, int page_size) {
    const int m = blockIdx.x;
    const int pos = positions[m];
    const int block = pos / page_size, at = pos % page_size;
    const int page = block < max_blocks ? block_table[(size_t)slots[m] * max_blocks + block] : -1;
    if (page < 0) return;                      // (no page: nothing is written)
    for (int i = threadIdx.x; i < kv_heads * key_dim; i += blockDim.x) {
        const int g = i / key_dim, d = i % key_dim;
        k_pages[(((size_t)page * kv_heads + g) * page_size + at) * key_dim + d] = k[(size_t)m * k_stride + i];
    }
    for (int i = threadIdx.x; i < kv_heads * value_dim; i += blockDim.x) {
        const int g = i / value_dim, d = i % value_dim;
        v_pages[(((size_t)page * kv_heads + g) * value_dim + d) * page_size + at] = v[(size_t)m * v_stride + i];
    }
}

// The rotation of a step's queries and keys and the write of its keys and values: a workgroup a token.  q is turned
// in place (columns of the projection's output); keys are turned on their way into the pages.  `rope` [positions,
// rot]: cosines in the first half of a row, sines in the second; every map of every head turns its first `rot`
// channels (rot <= head_dim, even), the others pass.  32-bit inside; rope null: nothing turns.
__global__ void diff_qkv_prep_kernel(elem_t* __restrict__ q, long q_stride, const elem_t* __restrict__ k, long k_stride,
                                     const elem_t* __restrict__ v, long v_stride, elem_t* __restrict__ k_pages,
                                     elem_t* __restrict__ v_pages, const int32_t* __restrict__ block_table, int max_blocks,
                                     const int32_t* __restrict__ slots, const int32_t* __restrict__ positions,
                                     const float* __restrict__ rope, int rot, int interleaved, int q_heads, int kv_heads,
                                     int head_dim, int value_dim, int page_size, int write_cache) {
    const int m = blockIdx.x;
    const int pos = positions[m];
    const int block = pos / page_size, at = pos % page_size;
    const int page = (write_cache && block < max_blocks) ? block_table[(size_t)slots[m] * max_blocks + block] : -1;
    const int half = rot / 2;
    const float* angle = rope != nullptr ? rope + (size_t)pos * rot : nullptr;
    // pairs of the queries: (head, map) x rot / 2
    if (angle != nullptr) {
        elem_t* qr = q + (size_t)m * q_stride;
        for (int i = threadIdx.x; i < q_heads * 2 * half; i += blockDim.x) {
            const int hm = i / half, j = i % half;
            const int d0 = interleaved ? 2 * j : j, d1 = interleaved ? 2 * j + 1 : j + half;
            elem_t* base = qr + (size_t)hm * head_dim;
            const float x = to_float(base[d0]), y = to_float(base[d1]), c = angle[j], s = angle[half + j];
            base[d0] = from_float<elem_t>(turn_x(x, y, c, s));
            base[d1] = from_float<elem_t>(turn_y(x, y, c, s));
        }
    }
    if (page < 0) return;                      // (no page: nothing is written)
    const int key_dim = 2 * head_dim;
    for (int i = threadIdx.x; i < kv_heads * key_dim; i += blockDim.x) {
        const int g = i / key_dim, d = i % key_dim, dm = d % head_dim;
        const elem_t* src = k + (size_t)m * k_stride;
        float val = to_float(src[i]);
        if (angle != nullptr && dm < rot) {
            const int j = interleaved ? dm / 2 : dm % half;
            const bool second = interleaved ? (dm & 1) : dm >= half;
            const int other = interleaved ? (second ? i - 1 : i + 1) : (second ? i - half : i + half);
            const float o = to_float(src[other]), c = angle[j], s = angle[half + j];
            val = second ? turn_y(o, val, c, s) : turn_x(val, o, c, s);
        }
        k_pages[(((size_t)page * kv_heads + g) * page_size + at) * key_dim + d] = from_float<elem_t>(val);
    }
    for (int i = threadIdx.x; i < kv_heads * value_dim; i += blockDim.x) {
        const int g = i / value_dim, d = i % value_dim;
        v_pages[(((size_t)page * kv_heads + g) * value_dim + d) * page_size + at] = v[(size_t)m * v_stride + i];
    }
}

__device__ __forceinline__ float query_temperature(int pos, float coef, float every) {
    return coef != 0.f ? 1.0f + coef * logf(floorf((float)(pos + 1) / every) + 1.0f) : 1.0f;
}

__global__ __launch_bounds__(64) void diff_attention_partial_kernel(DiffArgs a) {
    __shared__ float q_lds[256];
    __shared__ float k_lds[TILE_KEYS * (DIM_CHUNK + 1)];
    __shared__ float p_lds[TILE_KEYS];
    __shared__ long long k_off[TILE_KEYS];
    __shared__ long long v_off[TILE_KEYS];
    const int m = diff_row(a), hm = blockIdx.y, split = blockIdx.z;
    if (m < 0) return;
    const int head = hm >> 1, map = hm & 1;
    const int lane = threadIdx.x;
    const int D = a.head_dim, V = a.value_dim;
    const int kvh = head / (a.q_heads / a.kv_heads);
    const int pos = a.positions[m], slot = a.slots[m];
    int kbegin = first_key(a, pos), kend = pos + 1;
    if (a.max_splits > 1) {
        kbegin = max(kbegin, split * a.split_keys);
        kend = min(kend, (split + 1) * a.split_keys);
    }
    float* dst = a.partial + (((size_t)blockIdx.x * a.q_heads * 2 + hm) * a.max_splits + split) * (V + 2);
    if (kbegin >= kend) return;                // (a range beyond the token: the merge does not read it)
    for (int i = lane; i < D; i += 64) q_lds[i] = to_float(a.q[(size_t)m * a.q_stride + (size_t)hm * D + i]);
    const float factor = a.scale * query_temperature(pos, a.temp_coef, a.temp_every);
    float run_max = -INFINITY, run_sum = 0.f, acc[MAX_V_REGS];
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) acc[i] = 0.f;
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;
    for (int t0 = (kbegin / TILE_KEYS) * TILE_KEYS; t0 < kend; t0 += TILE_KEYS) {
        __syncthreads();
        {
            const int kp = t0 + lane;
            long long ko = -1, vo = -1;
            if (kp >= kbegin && kp < kend) {
                const int block = kp / a.page_size;
                const int page = block < a.max_blocks ? table[block] : -1;
                if (page >= 0) {
                    const long long head_page = (long long)page * a.kv_heads + kvh;
                    ko = (head_page * a.page_size + kp % a.page_size) * (2 * D) + (long long)map * D;
                    vo = head_page * V * a.page_size + kp % a.page_size;
                }
            }
            k_off[lane] = ko;
            v_off[lane] = vo;
        }
        float s = 0.f;
        for (int dc = 0; dc < D; dc += DIM_CHUNK) {
            const int dw = min(DIM_CHUNK, D - dc);
            __syncthreads();
            for (int i = lane; i < TILE_KEYS * dw; i += 64) {
                const int key = i / dw, d = i % dw;
                const long long off = k_off[key];
                k_lds[key * (DIM_CHUNK + 1) + d] = off >= 0 ? to_float(a.k_pages[off + dc + d]) : 0.f;
            }
            __syncthreads();
            const float* kr = k_lds + lane * (DIM_CHUNK + 1);
            float part = 0.f;
            for (int d = 0; d < dw; ++d) part += q_lds[dc + d] * kr[d];
            s += part;
        }
        const bool valid = k_off[lane] >= 0;
        s *= factor;
        if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
        if (!valid) s = -INFINITY;
        const float new_max = fmaxf(run_max, wave_max(s));
        const float p = (valid && new_max > -INFINITY) ? expf(s - new_max) : 0.f;
        const float corr = new_max > -INFINITY ? expf(run_max - new_max) : 1.f;
        run_sum = run_sum * corr + wave_sum(p);
        run_max = new_max;
#pragma unroll
        for (int i = 0; i < MAX_V_REGS; ++i) acc[i] *= corr;
        p_lds[lane] = p;
        __syncthreads();
        const int nkeys = min(TILE_KEYS, kend - t0);
        for (int key = 0; key < nkeys; ++key) {
            const long long off = v_off[key];
            if (off < 0) continue;
            const float pk = p_lds[key];
#pragma unroll
            for (int i = 0; i < MAX_V_REGS; ++i) {
                const int c = lane + 64 * i;
                if (c < V) acc[i] += pk * to_float(a.v_pages[off + (long long)c * a.page_size]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        if (c < V) dst[c] = acc[i];
    }
    if (lane == 0) {
        dst[V] = run_max;
        dst[V + 1] = run_sum;
    }
}

// One wavefront per (token, head): both maps merged over their key ranges, then the head's epilogue.
__global__ __launch_bounds__(64) void diff_attention_combine_kernel(DiffArgs a) {
    __shared__ float w_lds[COMBINE_MAX_SPLITS];
    __shared__ float l_lds[COMBINE_MAX_SPLITS];
    const int m = diff_row(a), head = blockIdx.y, lane = threadIdx.x;
    if (m < 0) return;
    const int V = a.value_dim;
    const int pos = a.positions[m];
    // the ranges that hold keys this token sees: from its first key's range to its own position's
    const int s0 = a.max_splits > 1 ? min(a.max_splits - 1, first_key(a, pos) / a.split_keys) : 0;
    const int n = (a.max_splits > 1 ? min(a.max_splits - 1, pos / a.split_keys) + 1 : 1) - s0;
    float maps[2][MAX_V_REGS];
    for (int map = 0; map < 2; ++map) {
        const float* base = a.partial + (((size_t)blockIdx.x * a.q_heads * 2 + head * 2 + map) * a.max_splits + s0) * (V + 2);
        float gmax = -INFINITY;
        __syncthreads();
        for (int s = lane; s < n; s += 64) {
            const float smax = base[(size_t)s * (V + 2) + V];
            w_lds[s] = smax;
            l_lds[s] = base[(size_t)s * (V + 2) + V + 1];
            gmax = fmaxf(gmax, smax);
        }
        gmax = wave_max(gmax);
        __syncthreads();
        for (int s = lane; s < n; s += 64) {
            const float smax = w_lds[s];
            w_lds[s] = smax > -INFINITY ? expf(smax - gmax) : 0.f;
        }
        __syncthreads();
        float den = 0.f;
        for (int s = 0; s < n; ++s) den += w_lds[s] * l_lds[s];
        float num[MAX_V_REGS];
#pragma unroll
        for (int i = 0; i < MAX_V_REGS; ++i) num[i] = 0.f;
        for (int s = 0; s < n; ++s) {
            const float w = w_lds[s];
            const float* p = base + (size_t)s * (V + 2);
#pragma unroll
            for (int i = 0; i < MAX_V_REGS; ++i) {
                const int c = lane + 64 * i;
                if (c < V) num[i] += w * p[c];
            }
        }
#pragma unroll
        for (int i = 0; i < MAX_V_REGS; ++i) maps[map][i] = den != 0.f ? num[i] / den : 0.f;
    }
    float o[MAX_V_REGS], ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        o[i] = c < V ? maps[0][i] - a.lam * maps[1][i] : 0.f;
        ss += o[i] * o[i];
    }
    ss = wave_sum(ss);
    const float unit = a.out_scale / sqrtf(ss / (float)V + a.eps);
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        if (c >= V) continue;
        float y = o[i] * unit;
        if (a.gate) y *= 1.0f / (1.0f + expf(-to_float(a.gate[(size_t)m * a.gate_stride + (size_t)head * V + c])));
        a.out[((size_t)m * a.q_heads + head) * V + c] = from_float<elem_t>(y);
    }
}

#if MLR_BF16
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
#define TKEYS 32
#define TILES_PAGE_CACHE 2048    // page ids of a workgroup's key range kept in LDS: the host keeps a range within them

// NCH: ceil(head_dim / 32) chunks of 32 channels a map; NDB: blocks of 16 value channels (value_dim <= 16 NDB).
// head_dim and value_dim multiples of 16, the page size a multiple of 8.
template <int NCH, int NDB>
__device__ __forceinline__ void diff_tiles_group(const DiffArgs& a, const int32_t* __restrict__ group_row0,
                                                 const int32_t* __restrict__ group_ntok, int col_heads, int wave_heads,
                                                 int token_blocks, int map_split, int grp, __bf16* k_lds, __bf16* v_lds,
                                                 int32_t* page_lds) {
    constexpr int KPITCH = 2 * 32 * NCH + 8;          // elements per key row in LDS (both maps)
    constexpr int VPITCH = TKEYS + 4;                 // elements per value channel row in LDS
    const int D = a.head_dim, V = a.value_dim, P = a.page_size;
    const int g = a.q_heads / a.kv_heads;
    // The 16 columns of a wavefront: `col_heads` query heads of the kv head side by side for each of 16 / col_heads
    // tokens (prompt portions: one head, 16 tokens; single tokens and short portions: up to four heads of each
    // token, so that one wavefront serves what four would).  The four wavefronts: `wave_heads` sets of heads x
    // `token_blocks` blocks of tokens; with `map_split` (partial results only) two sets of heads and blocks, wavefronts
    // 0 and 1 taking map 1 and wavefronts 2 and 3 map 2 of the same columns: half the chain of instructions a tile.
    const int heads_per_wg = col_heads * wave_heads;
    const int head_sets = (g + heads_per_wg - 1) / heads_per_wg;
    const int kvh = blockIdx.y / head_sets, head_set = blockIdx.y % head_sets;
    const int lane = threadIdx.x & 63, wave = map_split ? (int)((threadIdx.x >> 6) & 1) : (int)(threadIdx.x >> 6);
    const int my_map = threadIdx.x >> 7;              // (map_split only)
    const int col = lane & 15, b = lane >> 4;
    const int row0 = group_row0[grp], ntok = group_ntok[grp];
    const int slot = a.slots[row0], pos0 = a.positions[row0];
    const int tokens_per_wave = 16 / col_heads;
    const int head0 = (head_set * wave_heads + wave % wave_heads) * col_heads;      // the wavefront's first head in the set
    const int hh = head0 + col % col_heads;
    const int tblock = wave / wave_heads;
    const int head = kvh * g + hh;
    const int tok = tblock * tokens_per_wave + col / col_heads;
    const bool wave_active = tblock < token_blocks && head0 < g && tblock * tokens_per_wave < ntok;
    const bool col_valid = wave_active && col < tokens_per_wave * col_heads && hh < g && tok < ntok;
    const int pos = pos0 + tok;
    const int kend_c = col_valid ? pos + 1 : 0;       // keys this column sees: [kbeg_c, kend_c)
    const int kbeg_c = first_key(a, pos);
    const int ke = pos0 + ntok;                       // keys the workgroup walks: [first_key(pos0) in whole tiles, ke)
    const int wave_hi = wave_active ? pos0 + min(ntok, tblock * tokens_per_wave + tokens_per_wave) : 0;
    const int wave_first_kend = pos0 + tblock * tokens_per_wave + 1;
    // (first_key never decreases with the position: the wavefront's first token sees the earliest keys of its
    // columns, its last token's first key is seen by all of them)
    const int wave_first_kbeg = first_key(a, pos0 + tblock * tokens_per_wave);
    const int wave_last_kbeg = wave_active ? first_key(a, wave_hi - 1) : 0;
    const __bf16* q = reinterpret_cast<const __bf16*>(a.q);
    const __bf16* kp_base = reinterpret_cast<const __bf16*>(a.k_pages);
    const __bf16* vp_base = reinterpret_cast<const __bf16*>(a.v_pages);
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;

    bf16x8 qf[2][NCH];
#pragma unroll
    for (int map = 0; map < 2; ++map)
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int d0 = 32 * c + 8 * b;
            qf[map][c] = zero8;
            if (col_valid && d0 < D)
                qf[map][c] = *reinterpret_cast<const bf16x8*>(q + (size_t)(row0 + tok) * a.q_stride + (size_t)(head * 2 + map) * D + d0);
        }
    // scores in the base-2 domain; the cap as cap * tanh(x / cap) with tanh(y) = 1 - 2 / (exp(2 y) + 1)
    const float LOG2E = 1.44269504088896340736f;
    const float factor = a.scale * query_temperature(pos, a.temp_coef, a.temp_every);
    const bool capped = a.softcap > 0.f;
    const float pre = capped ? factor * (2.0f * LOG2E / a.softcap) : factor * LOG2E;
    const float cap2 = a.softcap * LOG2E;
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    floatx4 o[2][NDB];
#pragma unroll
    for (int map = 0; map < 2; ++map)
#pragma unroll
        for (int i = 0; i < NDB; ++i) o[map][i] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int k_chunks = TKEYS * (2 * D / 8);         // 16-byte chunks of a key tile: key-major
    const int v_chunks = V * (TKEYS / 8);             // of a value tile: channel-major, 8 keys each
    // with key ranges: this workgroup walks [split * split_keys, (split + 1) * split_keys) (multiples of 32) and
    // leaves partial results for the merge
    const int split = blockIdx.z;
    const int group_lo = (first_key(a, pos0) / TKEYS) * TKEYS;      // (the group's first token sees the earliest keys)
    const int k_lo = a.max_splits > 1 ? max(split * a.split_keys, group_lo) : group_lo;
    const int k_hi = a.max_splits > 1 ? min(ke, (split + 1) * a.split_keys) : ke;
    if (k_lo >= k_hi) return;                         // (a range beyond the group's keys: the merge does not read it)
    // page ids of the range first, so that a tile's loads do not wait for a load of the block table
    const int first_page = k_lo / P;                  // (the page that holds key k_lo)
    {
        const int n_pages = min(TILES_PAGE_CACHE, (k_hi + P - 1) / P - first_page);
        for (int i = threadIdx.x; i < n_pages; i += 256) page_lds[i] = first_page + i < a.max_blocks ? table[first_page + i] : -1;
        __syncthreads();
    }
    // (no load from the block table here: a global load behind a branch makes the compiler wait for every load in
    // flight, one tile's loads would then go out one after the other; the host keeps a range within the cache)
    const bool pow2 = (P & (P - 1)) == 0;
    const int pshift = __ffs(P) - 1;
    auto block_of = [&](int kp) { return pow2 ? kp >> pshift : kp / P; };
    auto within = [&](int kp) { return pow2 ? kp & (P - 1) : kp % P; };
    auto page_of = [&](int kp) {
        const int page = page_lds[min(max(block_of(kp) - first_page, 0), TILES_PAGE_CACHE - 1)];
        return kp < k_hi ? page : -1;
    };
    // what a thread stages does not change from tile to tile
    constexpr int KST = NCH, VST = (NDB + 3) / 4;     // 16-byte chunks a thread stages per tile
    int k_key[KST], k_goff[KST], k_loff[KST], v_ch[VST], v_key[VST], v_loff[VST];
    bool k_mine[KST], v_mine[VST];
#pragma unroll
    for (int i = 0; i < KST; ++i) {
        k_mine[i] = (int)threadIdx.x + 256 * i < k_chunks;
        const int ci = min((int)threadIdx.x + 256 * i, k_chunks - 1);
        const int key = ci / (2 * D / 8), ch = 8 * (ci % (2 * D / 8)), map = ch >= D ? 1 : 0;
        k_key[i] = key;
        k_goff[i] = ch;
        // (map m's channel d goes to column m * 32 NCH + d, so that both maps start a row of chunks)
        k_loff[i] = key * KPITCH + map * 32 * NCH + (ch - map * D);
    }
#pragma unroll
    for (int i = 0; i < VST; ++i) {
        v_mine[i] = (int)threadIdx.x + 256 * i < v_chunks;
        const int ci = min((int)threadIdx.x + 256 * i, v_chunks - 1);
        v_ch[i] = ci >> 2;
        v_key[i] = 8 * (ci & 3);
        v_loff[i] = (ci >> 2) * VPITCH + 8 * (ci & 3);
    }
    struct Staged {                                   // one tile on its way: registers between memory and LDS
        bf16x8 k[KST], v[VST];
        int tb, ok;                                   // bit i: chunk i of the keys, bit 16 + i: of the values, is there
    };
    // global -> registers, no branch around a load (a load behind a branch makes the compiler wait for every load in
    // flight): addresses are clamped to memory that exists, what must read as zero is zeroed on the way to LDS
    auto fetch = [&](int tb, Staged& st) {
        st.tb = tb;
        st.ok = 0;
#pragma unroll
        for (int i = 0; i < KST; ++i) {
            const int kp = tb + k_key[i];
            const int page = page_of(kp);
            if (page >= 0 && k_mine[i]) st.ok |= 1 << i;
            st.k[i] = *reinterpret_cast<const bf16x8*>(kp_base + (((size_t)max(page, 0) * a.kv_heads + kvh) * P + within(kp)) * (2 * D) + k_goff[i]);
        }
#pragma unroll
        for (int i = 0; i < VST; ++i) {
            const int kp = tb + v_key[i];
            const int page = page_of(kp);
            if (page >= 0 && v_mine[i]) st.ok |= 1 << (16 + i);
            st.v[i] = *reinterpret_cast<const bf16x8*>(vp_base + (((size_t)max(page, 0) * a.kv_heads + kvh) * V + v_ch[i]) * P + within(kp));
        }
    };
    auto stash = [&](const Staged& st) {              // registers -> LDS
#pragma unroll
        for (int i = 0; i < KST; ++i) {
            if (!k_mine[i]) continue;
            *reinterpret_cast<bf16x8*>(&k_lds[k_loff[i]]) = ((st.ok >> i) & 1) ? st.k[i] : zero8;
        }
#pragma unroll
        for (int i = 0; i < VST; ++i) {
            if (!v_mine[i]) continue;
            bf16x8 v = ((st.ok >> (16 + i)) & 1) ? st.v[i] : zero8;
            const int key0 = st.tb + v_key[i];
            if (key0 + 8 > k_hi) {
#pragma unroll
                for (int e = 0; e < 8; ++e)           // keys that are not written yet count as zero
                    if (key0 + e >= k_hi) v[e] = (__bf16)0.f;
            }
            *reinterpret_cast<bf16x4*>(&v_lds[v_loff[i]]) = bf16x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<bf16x4*>(&v_lds[v_loff[i] + 4]) = bf16x4{v[4], v[5], v[6], v[7]};
        }
    };
    auto compute = [&](int tb) {
        if (!wave_active || tb >= wave_hi || tb + TKEYS <= wave_first_kbeg) return;
        const bool interior = tb + TKEYS <= wave_first_kend && tb >= wave_last_kbeg;
#pragma unroll
        for (int map = 0; map < 2; ++map) {
            if (map_split && map != my_map) continue;
            floatx4 s[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                s[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    bf16x8 kf = zero8;                // (channels at and beyond head_dim were never staged)
                    if (32 * c + 8 * b < D)
                        kf = *reinterpret_cast<const bf16x8*>(&k_lds[(16 * j + col) * KPITCH + map * 32 * NCH + 32 * c + 8 * b]);
                    s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[map][c], s[j], 0, 0, 0);
                }
            }
            float sv[2][4];
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float x = s[j][r] * pre;
                    if (capped) {
                        const float e = __builtin_amdgcn_exp2f(x);                    // exp(2 s / cap)
                        x = cap2 - 2.0f * cap2 * __builtin_amdgcn_rcpf(e + 1.0f);
                    }
                    const int key = tb + 16 * j + 4 * b + r;
                    sv[j][r] = (interior || (key < kend_c && key >= kbeg_c)) ? x : -INFINITY;
                }
            float tile_max = fmaxf(fmaxf(fmaxf(sv[0][0], sv[0][1]), fmaxf(sv[0][2], sv[0][3])),
                                   fmaxf(fmaxf(sv[1][0], sv[1][1]), fmaxf(sv[1][2], sv[1][3])));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, MLR_WAVE));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, MLR_WAVE));
            // (the running maximum rarely moves after the first tiles: rescale only when it does, for any column)
            if (__builtin_amdgcn_ballot_w64(tile_max > m_run[map]) != 0) {
                const float m_new = fmaxf(m_run[map], tile_max);
                const float corr = m_new > -INFINITY ? __builtin_amdgcn_exp2f(m_run[map] - m_new) : 1.f;
                l_run[map] *= corr;
#pragma unroll
                for (int db = 0; db < NDB; ++db) o[map][db] *= corr;
                m_run[map] = m_new;
            }
            const float m_use = fmaxf(m_run[map], -1e30f);
            bf16x8 pf;
            float psum = 0.f;
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float p = __builtin_amdgcn_exp2f(sv[j][r] - m_use);
                    psum += p;
                    pf[4 * j + r] = (__bf16)p;
                }
            l_run[map] += psum;
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                if (16 * db >= V) break;
                const __bf16* vrow = &v_lds[(16 * db + col) * VPITCH];
                const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(vrow + 4 * b);
                const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(vrow + 16 + 4 * b);
                const bf16x8 vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                o[map][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[map][db], 0, 0, 0);
            }
        }
    };
    // Two tiles are on their way from memory while one is multiplied: with one, a workgroup's time a tile is the
    // memory's answer time.  (Fetches are unconditional, clamped to the last tile.)
    const int tb_last = k_lo + ((k_hi - k_lo - 1) / TKEYS) * TKEYS;
    Staged sa, sb;
    fetch(k_lo, sa);
    fetch(min(k_lo + TKEYS, tb_last), sb);
    for (int tb = k_lo; tb < k_hi; tb += 2 * TKEYS) {
        __syncthreads();                              // the tile before has been read
        stash(sa);
        __syncthreads();
        fetch(min(tb + 2 * TKEYS, tb_last), sa);
        compute(tb);
        if (tb + TKEYS >= k_hi) break;
        __syncthreads();
        stash(sb);
        __syncthreads();
        fetch(min(tb + 3 * TKEYS, tb_last), sb);
        compute(tb + TKEYS);
    }
#pragma unroll
    for (int map = 0; map < 2; ++map) {
        l_run[map] += __shfl_xor(l_run[map], 16, MLR_WAVE);
        l_run[map] += __shfl_xor(l_run[map], 32, MLR_WAVE);
    }
    if (a.partial != nullptr) {
        // (max, sum, weighted values) of this key range, the maximum back in the natural domain
        if (!col_valid) return;
        const size_t place = (size_t)grp * a.group_tokens + tok;
#pragma unroll
        for (int map = 0; map < 2; ++map) {
            if (map_split && map != my_map) continue;
            float* dst = a.partial + ((place * a.q_heads * 2 + head * 2 + map) * a.max_splits + split) * (V + 2);
#pragma unroll
            for (int db = 0; db < NDB; ++db) {
                if (16 * db >= V) break;
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[16 * db + 4 * b + r] = o[map][db][r];
            }
            if (b == 0) {
                dst[V] = m_run[map] * 0.69314718055994530942f;
                dst[V + 1] = l_run[map];
            }
        }
        return;
    }
    // the head's epilogue: lane (col, b) holds channels 16 db + 4 b + r of its column
    const float inv1 = l_run[0] != 0.f ? 1.0f / l_run[0] : 0.f, inv2 = l_run[1] != 0.f ? 1.0f / l_run[1] : 0.f;
    float ss = 0.f;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        if (16 * db >= V) break;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float d = o[0][db][r] * inv1 - a.lam * (o[1][db][r] * inv2);
            o[0][db][r] = d;
            ss += d * d;
        }
    }
    ss += __shfl_xor(ss, 16, MLR_WAVE);
    ss += __shfl_xor(ss, 32, MLR_WAVE);
    if (!col_valid) return;
    const float unit = a.out_scale / sqrtf(ss / (float)V + a.eps);
    __bf16* dst = reinterpret_cast<__bf16*>(a.out) + ((size_t)(row0 + tok) * a.q_heads + head) * V;
    const __bf16* gate = a.gate ? reinterpret_cast<const __bf16*>(a.gate) + (size_t)(row0 + tok) * a.gate_stride + (size_t)head * V : nullptr;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
        if (16 * db >= V) break;
        bf16x4 w4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float y = o[0][db][r] * unit;
            if (gate) y *= 1.0f / (1.0f + __expf(-(float)gate[16 * db + 4 * b + r]));
            w4[r] = (__bf16)y;
        }
        *reinterpret_cast<bf16x4*>(dst + 16 * db + 4 * b) = w4;
    }
}

template <int NCH, int NDB>
__global__ __launch_bounds__(256) void diff_attention_tiles_kernel(DiffArgs a, const int32_t* __restrict__ group_row0,
                                                                   const int32_t* __restrict__ group_ntok, int groups,
                                                                   int col_heads, int wave_heads, int token_blocks,
                                                                   int map_split) {
    __shared__ __attribute__((aligned(16))) __bf16 k_lds[TKEYS * (2 * 32 * NCH + 8)];
    __shared__ __attribute__((aligned(16))) __bf16 v_lds[16 * NDB * (TKEYS + 4)];
    __shared__ int32_t page_lds[TILES_PAGE_CACHE];
    // (the longest groups of a prompt first: the workgroups that start last are the short ones)
    diff_tiles_group<NCH, NDB>(a, group_row0, group_ntok, col_heads, wave_heads, token_blocks, map_split,
                               groups - 1 - (int)blockIdx.x, k_lds, v_lds, page_lds);
}

template <int NCH>
static int launch_tiles(const DiffArgs& a, const int32_t* row0, const int32_t* ntok, int groups, int ch, int wh, int tbw,
                        int ms, hipStream_t stream) {
    const int g = a.q_heads / a.kv_heads;
    dim3 grid(groups, a.kv_heads * ((g + ch * wh - 1) / (ch * wh)), a.max_splits);
    const int ndb = (a.value_dim + 15) / 16;
    if (ndb <= 2) diff_attention_tiles_kernel<NCH, 2><<<grid, 256, 0, stream>>>(a, row0, ntok, groups, ch, wh, tbw, ms);
    else if (ndb <= 4) diff_attention_tiles_kernel<NCH, 4><<<grid, 256, 0, stream>>>(a, row0, ntok, groups, ch, wh, tbw, ms);
    else diff_attention_tiles_kernel<NCH, 8><<<grid, 256, 0, stream>>>(a, row0, ntok, groups, ch, wh, tbw, ms);
    return (int)hipGetLastError();
}
#endif

extern "C" {

int mlr_diff_kv_write(const void* k, long k_stride, const void* v, long v_stride, void* k_pages, void* v_pages,
                      const int32_t* block_table, int max_blocks, const int32_t* slots, const int32_t* positions, int rows,
                      int kv_heads, int key_dim, int value_dim, int page_size, hipStream_t stream) {
    if (rows <= 0) return 0;
    diff_kv_write_kernel<<<rows, 256, 0, stream>>>((const elem_t*)k, k_stride, (const elem_t*)v, v_stride, (elem_t*)k_pages,
                                                   (elem_t*)v_pages, block_table, max_blocks, slots, positions, kv_heads,
                                                   key_dim, value_dim, page_size);
    return (int)hipGetLastError();
}

int mlr_diff_qkv_prep(void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride, void* k_pages,
                      void* v_pages, const int32_t* block_table, int max_blocks, const int32_t* slots,
                      const int32_t* positions, const float* rope, int rot, int interleaved, int rows, int q_heads,
                      int kv_heads, int head_dim, int value_dim, int page_size, int write_cache, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (rope != nullptr && (rot < 2 || rot % 2 != 0 || rot > head_dim)) return -1;
    diff_qkv_prep_kernel<<<rows, 256, 0, stream>>>((elem_t*)q, q_stride, (const elem_t*)k, k_stride, (const elem_t*)v, v_stride,
                                                   (elem_t*)k_pages, (elem_t*)v_pages, block_table, max_blocks, slots,
                                                   positions, rope, rot, interleaved, q_heads, kv_heads, head_dim, value_dim,
                                                   page_size, write_cache);
    return (int)hipGetLastError();
}

int mlr_diff_attention(const void* q, long q_stride, const void* k_pages, const void* v_pages, const int32_t* block_table,
                       int max_blocks, const int32_t* slots, const int32_t* positions, const void* gate, long gate_stride,
                       void* out, float* partial, int rows, int q_heads, int kv_heads, int head_dim, int value_dim,
                       int page_size, float scale, float softcap, float temp_coef, float temp_every, float lam,
                       float out_scale, float eps, int split_keys, int max_splits, const int32_t* group_first,
                       const int32_t* group_count, int groups, int group_tokens, int mask_kind, int mask_size,
                       hipStream_t stream) {
    // (with groups: `rows` = groups * group_tokens places, of which those beyond a group's count stay idle)
    if (group_first != nullptr) rows = groups * group_tokens;
    if (rows <= 0) return 0;
    if (head_dim > 256 || value_dim > 64 * MAX_V_REGS || q_heads % kv_heads != 0 || partial == nullptr) return -1;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 1 && (split_keys <= 0 || split_keys % TILE_KEYS != 0 || max_splits > COMBINE_MAX_SPLITS)) return -2;
    if (temp_coef != 0.f && !(temp_every > 0.f)) return -3;
    if (mask_kind < MASK_NONE || mask_kind > MASK_CHUNK || (mask_kind != MASK_NONE && mask_size < 1)) return -5;
    DiffArgs a{(const elem_t*)q, q_stride, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots, positions,
               (const elem_t*)gate, gate_stride, (elem_t*)out, partial, max_blocks, q_heads, kv_heads, head_dim, value_dim,
               page_size, split_keys, max_splits, scale, softcap, temp_coef, temp_every, lam, out_scale, eps,
               group_first, group_count, group_tokens, mask_kind, mask_size};
    diff_attention_partial_kernel<<<dim3(rows, q_heads * 2, max_splits), 64, 0, stream>>>(a);
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    diff_attention_combine_kernel<<<dim3(rows, q_heads), 64, 0, stream>>>(a);
    return (int)hipGetLastError();
}

// Groups of consecutive tokens of one request on the matrix cores (bfloat16): prompt portions in groups of up to
// 16 * (4 / min(4, q_heads / kv_heads)) tokens, single tokens and short portions in smaller ones.  `group_tokens`:
// the most tokens of a group.  With max_splits > 1 every group's keys are cut into ranges of split_keys (a
// multiple of 64) whose partial results [groups * group_tokens, q_heads * 2, max_splits, value_dim + 2] are merged
// by the kernel that also serves the scalar path.  `max_context`: no token of the step lies at or beyond it.
// Returns -10 where the sizes are not taken.
int mlr_diff_attention_tiles(const void* q, long q_stride, const void* k_pages, const void* v_pages,
                             const int32_t* block_table, int max_blocks, const int32_t* slots, const int32_t* positions,
                             const void* gate, long gate_stride, void* out, float* partial, const int32_t* group_row0,
                             const int32_t* group_ntok, int groups, int group_tokens, int q_heads, int kv_heads,
                             int head_dim, int value_dim, int page_size, float scale, float softcap, float temp_coef,
                             float temp_every, float lam, float out_scale, float eps, int split_keys, int max_splits,
                             int max_context, int mask_kind, int mask_size, hipStream_t stream) {
#if MLR_BF16
    if (groups <= 0) return 0;
    if (mask_kind < MASK_NONE || mask_kind > MASK_CHUNK || (mask_kind != MASK_NONE && mask_size < 1)) return -5;
    // (behind a mask a workgroup walks the keys of its tokens' window or block only)
    if (mask_kind != MASK_NONE && mask_size + group_tokens + 2 * TILE_KEYS < max_context)
        max_context = mask_size + group_tokens + 2 * TILE_KEYS;
    // the keys one workgroup walks (a range, or without ranges the longest context of the step) lie in at most
    // TILES_PAGE_CACHE pages, whose ids it keeps in LDS
    if (((max_splits > 1 ? split_keys : max_context) + page_size - 1) / page_size + 1 > TILES_PAGE_CACHE) return -4;
    if (head_dim % 16 != 0 || head_dim > 128 || value_dim % 16 != 0 || value_dim > 128 || page_size % 8 != 0 ||
        q_heads % kv_heads != 0 || q_stride % 8 != 0 || (gate != nullptr && gate_stride % 4 != 0)) return -10;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 1 && (partial == nullptr || split_keys <= 0 || split_keys % TILE_KEYS != 0 ||
                           max_splits > COMBINE_MAX_SPLITS)) return -2;
    // (partial given with one range: the kernel still leaves partial results and the merge kernel finishes the head)
    const int g = q_heads / kv_heads;
    // groups of up to four tokens: up to four heads of a token side by side in a wavefront's columns; longer groups
    // (prompt portions): a head a wavefront, 16 tokens in its columns
    const int ch = group_tokens <= 4 ? (g < 4 ? g : 4) : 1;
    const int sets = (g + ch - 1) / ch;
    // (with partial results, small groups give each map wavefronts of its own: two layout places instead of four)
    const int ms = (group_tokens <= 4 && partial != nullptr) ? 1 : 0;
    const int places = ms ? 2 : 4;
    const int wh = sets < places ? sets : places, tbw = places / wh;
    if (group_tokens < 1 || group_tokens > (16 / ch) * tbw) return -3;
    DiffArgs a{(const elem_t*)q, q_stride, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots, positions,
               (const elem_t*)gate, gate_stride, (elem_t*)out, partial, max_blocks, q_heads, kv_heads, head_dim, value_dim,
               page_size, split_keys, max_splits, scale, softcap, temp_coef, temp_every, lam, out_scale, eps,
               group_row0, group_ntok, group_tokens, mask_kind, mask_size};
    const int nch = (head_dim + 31) / 32;
    int err;
    if (nch == 1) err = launch_tiles<1>(a, group_row0, group_ntok, groups, ch, wh, tbw, ms, stream);
    else if (nch == 2) err = launch_tiles<2>(a, group_row0, group_ntok, groups, ch, wh, tbw, ms, stream);
    else err = launch_tiles<4>(a, group_row0, group_ntok, groups, ch, wh, tbw, ms, stream);
    if (err != 0 || partial == nullptr) return err;
    diff_attention_combine_kernel<<<dim3(groups * group_tokens, q_heads), 64, 0, stream>>>(a);
    return (int)hipGetLastError();
#else
    return -10;
#endif
}

}  // extern "C"
