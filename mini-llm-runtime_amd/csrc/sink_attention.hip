// Softmax attention with a sink and a mask rule over the paged cache, for mixers whose keys and values have
// sizes of their own, and the row kernels that prepare their queries, keys and values.
//
// A query at position p of a request sees the keys lo(p) .. p of the same request:
//   MASK_ALL     lo = 0
//   MASK_WINDOW  lo = max(0, p - size + 1)         (itself and the size - 1 tokens before it)
//   MASK_CHUNK   lo = floor(p / size) * size        (the keys of its own block of `size` positions)
// positions counted from the request's first token, never from where a step cut it.  The softmax's denominator
// holds one more summand, exp(sink[head]) (no key, no value, not scaled); sink == null: none.
// score = (q . k) * scale.  Scores, the softmax and its sums are 32-bit.
//
// Cache of one layer: key rows k_pages[page][kv_head][place in page][k_row] of which the first key_dim channels
// are the key, value rows v_pages[page][kv_head][place][v_row] of which the first value_dim channels are the
// value; both row-major.  The value rows may BE the key rows (v_pages == k_pages, v_row == k_row): a latent
// vector that serves as the first channels of the key and as the value.  Query head h reads kv head
// h / (q_heads / kv_heads).
//
// `sink_attention_kernel`: one wavefront per (token, head); tiles of 64 keys that start at multiples of 64 of the
// absolute position, so the order of a token's sums follows from its own position alone, never from the batch
// around it or from how its request was cut into steps.  The float engine's only attention, and the bfloat16
// engine's for sizes that the matrix-core kernel does not take.
// `sink_attention_tiles_kernel` (bfloat16): the same on the matrix cores, see there.
#include "common.h"

#define MASK_ALL 0
#define MASK_WINDOW 1
#define MASK_CHUNK 2

#define TILE_KEYS 64
#define DIM_CHUNK 64
#define MAX_KEY_DIM 2048
#define MAX_V_REGS 16           // value_dim <= 64 * MAX_V_REGS

struct SinkArgs {
    const elem_t* q; long q_stride;            // q[m * q_stride + head * key_dim + d]
    const elem_t* k_pages; long k_row;
    const elem_t* v_pages; long v_row;
    const int32_t* block_table; const int32_t* slots; const int32_t* positions;
    const float* sink;                         // [q_heads] or null
    elem_t* out; long out_stride;              // out[m * out_stride + head * value_dim + c]
    int max_blocks, q_heads, kv_heads, key_dim, value_dim, page_size, mask_kind, mask_size;
    float scale;
    // key ranges over several workgroups (the matrix-core kernel): workgroup z of a group takes split_keys keys from
    // the group's first tile on and leaves (unnormalised values, maximum, sum) in partial[((g * tokens + i) * q_heads +
    // head) * splits + z][value_dim + 4] for token i of group g; null: one workgroup walks every key and writes out
    float* partial; int split_keys, splits, group_tokens;
};

__device__ __forceinline__ int first_seen(int pos, int kind, int size) {
    if (kind == MASK_WINDOW) return max(0, pos - size + 1);
    if (kind == MASK_CHUNK) return (pos / size) * size;
    return 0;
}

__global__ __launch_bounds__(64) void sink_attention_kernel(SinkArgs a) {
    __shared__ float q_lds[MAX_KEY_DIM];
    __shared__ float k_lds[TILE_KEYS * (DIM_CHUNK + 1)];
    __shared__ float p_lds[TILE_KEYS];
    __shared__ long long row_of[TILE_KEYS];
    const int m = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int D = a.key_dim, V = a.value_dim;
    const int kvh = head / (a.q_heads / a.kv_heads);
    const int pos = a.positions[m], slot = a.slots[m];
    const int kbegin = first_seen(pos, a.mask_kind, a.mask_size), kend = pos + 1;
    for (int i = lane; i < D; i += 64) q_lds[i] = to_float(a.q[(size_t)m * a.q_stride + (size_t)head * D + i]);
    float run_max = -INFINITY, run_sum = 0.f, acc[MAX_V_REGS];
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) acc[i] = 0.f;
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;
    for (int t0 = (kbegin / TILE_KEYS) * TILE_KEYS; t0 < kend; t0 += TILE_KEYS) {
        __syncthreads();
        {
            const int kp = t0 + lane;
            long long r = -1;
            if (kp >= kbegin && kp < kend) {
                const int block = kp / a.page_size;
                const int page = block < a.max_blocks ? table[block] : -1;
                if (page >= 0) r = ((long long)page * a.kv_heads + kvh) * a.page_size + kp % a.page_size;
            }
            row_of[lane] = r;
        }
        float s = 0.f;
        for (int dc = 0; dc < D; dc += DIM_CHUNK) {
            const int dw = min(DIM_CHUNK, D - dc);
            __syncthreads();
            for (int i = lane; i < TILE_KEYS * dw; i += 64) {
                const int key = i / dw, d = i % dw;
                const long long r = row_of[key];
                k_lds[key * (DIM_CHUNK + 1) + d] = r >= 0 ? to_float(a.k_pages[r * a.k_row + dc + d]) : 0.f;
            }
            __syncthreads();
            const float* kr = k_lds + lane * (DIM_CHUNK + 1);
            float part = 0.f;
            for (int d = 0; d < dw; ++d) part += q_lds[dc + d] * kr[d];
            s += part;
        }
        const bool valid = row_of[lane] >= 0;
        s = valid ? s * a.scale : -INFINITY;
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
            const long long r = row_of[key];
            if (r < 0) continue;
            const float pk = p_lds[key];
            const elem_t* vr = a.v_pages + r * a.v_row;
#pragma unroll
            for (int i = 0; i < MAX_V_REGS; ++i) {
                const int c = lane + 64 * i;
                if (c < V) acc[i] += pk * to_float(vr[c]);
            }
        }
    }
    // the sink: one more summand of the denominator
    float top = run_max, den = run_sum, scale_acc = 1.f;
    if (a.sink != nullptr) {
        const float sk = a.sink[head];
        top = fmaxf(run_max, sk);
        scale_acc = run_max > -INFINITY ? expf(run_max - top) : 0.f;
        den = run_sum * scale_acc + expf(sk - top);
    }
    const float inv = den > 0.f ? scale_acc / den : 0.f;
    elem_t* dst = a.out + (size_t)m * a.out_stride + (size_t)head * V;
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        if (c < V) dst[c] = from_float<elem_t>(acc[i] * inv);
    }
}

// ---------------------------------------------------------------------------------------------------------
// Queries, keys and values of a grouped-query attention from the stacked projection's output
// proj[m] = [q_heads * key_dim | kv_heads * key_dim | kv_heads * value_dim]: the projection's bias added (null:
// none); q and k normed per head over key_dim (x / sqrt(mean(x^2) + eps) * weight, the weight shared by the
// heads; null: no weight) before the rotation (norm_mode 1), after it (norm_mode 2) or not at all (0); the first
// rot_dim channels of a head turned by the token's position with cos = table[p][j], sin = table[p][rot_dim / 2 + j]
// in pairs (j, j + rot_dim / 2) or, `interleaved`, (2 j, 2 j + 1) (table null: no rotation);
// q to q_out [m, q_heads * key_dim], k and v into their pages.  One wavefront a head; 32-bit throughout.
__device__ __forceinline__ float turned_channel(const float* x, int d, const float* cs, int rot_dim, int interleaved) {
    if (cs == nullptr || d >= rot_dim) return x[d];
    const int half = rot_dim >> 1;
    if (interleaved) {
        const int j = d >> 1;
        const float c = cs[j], s = cs[half + j];
        return (d & 1) ? turn_y(x[d - 1], x[d], c, s) : turn_x(x[d], x[d + 1], c, s);
    }
    const int j = d < half ? d : d - half;
    const float c = cs[j], s = cs[half + j];
    return d < half ? turn_x(x[d], x[d + half], c, s) : turn_y(x[d - half], x[d], c, s);
}

__global__ __launch_bounds__(64) void sink_qkv_prep_kernel(
    const elem_t* __restrict__ proj, long ld, const float* __restrict__ bias, elem_t* __restrict__ q_out,
    elem_t* __restrict__ k_pages, long k_row, elem_t* __restrict__ v_pages, long v_row,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ positions, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
    float eps, const float* __restrict__ rope, int rot_dim, int q_heads, int kv_heads, int key_dim, int value_dim,
    int page_size, int write_cache, int norm_mode, int interleaved) {
    __shared__ float x_lds[MAX_KEY_DIM];
    const int m = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[m], slot = slots[m];
    long long cache_row = -1;
    if (unit >= q_heads) {
        if (!write_cache) return;
        const int block = pos / page_size;
        const int page = block < max_blocks ? block_table[(size_t)slot * max_blocks + block] : -1;
        if (page < 0) return;                  // (no page: nothing is written)
        const int kvh = unit < q_heads + kv_heads ? unit - q_heads : unit - q_heads - kv_heads;
        cache_row = ((long long)page * kv_heads + kvh) * page_size + pos % page_size;
    }
    if (unit >= q_heads + kv_heads) {          // a value head: bias, into its page
        const long off = (long)(q_heads + kv_heads) * key_dim + (long)(unit - q_heads - kv_heads) * value_dim;
        for (int c = lane; c < value_dim; c += 64)
            v_pages[cache_row * v_row + c] =
                from_float<elem_t>(to_float(proj[(size_t)m * ld + off + c]) + (bias ? bias[off + c] : 0.f));
        return;
    }
    const long off = (long)unit * key_dim;
    const float* w = unit < q_heads ? q_norm_w : k_norm_w;
    float sum = 0.f;
    for (int d = lane; d < key_dim; d += 64) {
        const float x = to_float(proj[(size_t)m * ld + off + d]) + (bias ? bias[off + d] : 0.f);
        x_lds[d] = x;
        sum += x * x;
    }
    if (norm_mode == 1) {
        sum = wave_sum(sum);
        const float r = 1.0f / sqrtf(sum / (float)key_dim + eps);
        for (int d = lane; d < key_dim; d += 64) x_lds[d] = (x_lds[d] * r) * (w != nullptr ? w[d] : 1.0f);
    }
    __syncthreads();
    elem_t* dst = unit < q_heads ? q_out + ((size_t)m * q_heads + unit) * key_dim : k_pages + cache_row * k_row;
    const float* cs = rope ? rope + (size_t)pos * rot_dim : nullptr;
    float r_after = 1.0f;
    if (norm_mode == 2) {                       // the root mean square of the head as it is after the rotation
        float turned = 0.f;
        for (int d = lane; d < key_dim; d += 64) {
            const float y = turned_channel(x_lds, d, cs, rot_dim, interleaved);
            turned += y * y;
        }
        turned = wave_sum(turned);
        r_after = 1.0f / sqrtf(turned / (float)key_dim + eps);
    }
    for (int d = lane; d < key_dim; d += 64) {
        float y = turned_channel(x_lds, d, cs, rot_dim, interleaved);
        if (norm_mode == 2) y = (y * r_after) * (w != nullptr ? w[d] : 1.0f);
        dst[d] = from_float<elem_t>(y);
    }
}

// Latent attention's row work.  q_src[m] = [heads * (dim + rot)]: per head `dim` plain and `rot` rotated query
// channels; kv_src[m] = [rank + rot]: the latent part (`rank` channels) and the one rotated key part all heads
// share (the two may be column blocks of one projection's output).
//   units 0 .. heads - 1: the head's rotated query channels, turned by the token's position (pairs
//     (j, j + rot / 2) or, `interleaved`, (2 j, 2 j + 1)), to q_out[m][head][rank .. rank + rot) -- the plain
//     channels reach q_out[m][head][0 .. rank) through the key up-projection, which is another kernel's work;
//   unit heads: the latent part normed over its `rank` channels (x / sqrt(mean(x^2) + eps) * weight) and the
//     rotated key part turned, into the token's cache row [rank + rot].
__device__ __forceinline__ void turn_part(const elem_t* src, elem_t* dst, const float* cs, int rot, int interleaved, int lane) {
    const int half = rot >> 1;
    for (int j = lane; j < half; j += 64) {
        const int a = interleaved ? 2 * j : j, b = interleaved ? 2 * j + 1 : j + half;
        const float u = to_float(src[a]), v = to_float(src[b]);
        dst[a] = from_float<elem_t>(turn_x(u, v, cs[j], cs[half + j]));
        dst[b] = from_float<elem_t>(turn_y(u, v, cs[j], cs[half + j]));
    }
}

__global__ __launch_bounds__(64) void latent_prep_kernel(
    const elem_t* __restrict__ q_src, long q_ld, const elem_t* __restrict__ kv_src, long kv_ld, elem_t* __restrict__ q_out,
    elem_t* __restrict__ pages, long row_width, const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ slots, const int32_t* __restrict__ positions, const float* __restrict__ norm_w, float eps,
    const float* __restrict__ rope, int heads, int dim, int rot, int rank, int page_size, int write_cache, int interleaved) {
    const int m = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[m];
    const float* cs = rope + (size_t)pos * rot;
    if (unit < heads) {
        turn_part(q_src + (size_t)m * q_ld + (size_t)unit * (dim + rot) + dim,
                  q_out + ((size_t)m * heads + unit) * (rank + rot) + rank, cs, rot, interleaved, lane);
        return;
    }
    if (!write_cache) return;
    const int block = pos / page_size;
    const int page = block < max_blocks ? block_table[(size_t)slots[m] * max_blocks + block] : -1;
    if (page < 0) return;
    elem_t* dst = pages + ((long long)page * page_size + pos % page_size) * row_width;
    const elem_t* src = kv_src + (size_t)m * kv_ld;
    float sum = 0.f;
    for (int d = lane; d < rank; d += 64) {
        const float x = to_float(src[d]);
        sum += x * x;
    }
    sum = wave_sum(sum);
    const float r = 1.0f / sqrtf(sum / (float)rank + eps);
    for (int d = lane; d < rank; d += 64) dst[d] = from_float<elem_t>((to_float(src[d]) * r) * norm_w[d]);
    turn_part(src + rank, dst + rank, cs, rot, interleaved, lane);
}

#if MLR_BF16
// ---------------------------------------------------------------------------------------------------------
// The same attention on the matrix cores (bfloat16 engine; keys in multiples of 8 channels up to 576, values in
// multiples of 16 up to 512): prompt portions and single tokens.
//
// A workgroup (4 wavefronts) serves ONE group of consecutive tokens of a request and up to `head_block` query heads
// of one kv head: 64 columns (token, head), token = column / head_block.  It walks the keys that its tokens see,
// from the first key of the group's first token to the last token's own position, in tiles of 32 keys at absolute
// multiples of 32; a tile's key rows are staged once through LDS for all its columns (row-major for the scores,
// and the value channels transposed, [channel][key], for the second product: 16-byte reads of eight keys of one
// channel), the next tile's rows on their way from memory into registers meanwhile.  A thread stages 16 bytes (eight
// channels of one key); consecutive lanes take consecutive KEYS, so that the eight 2-byte writes that transpose
// them land in different LDS banks (lanes that take consecutive channels of one key all meet in two banks, which
// made a tile's staging ten times as long as its products).  Where the value rows ARE the
// key rows they are read once.  Rows outside the range, or without a page, are staged as zeros.
//   S^T = K Q^T with v_mfma_f32_16x16x32_bf16: row i of the instruction's first operand is tile key
//   8 (i / 4) + 4 s + i % 4 of half-tile s, so that a lane ends up with the scores of the eight CONSECUTIVE keys
//   8 b .. 8 b + 7 (b = lane / 16) of its column (lane % 16): the probabilities are the second product's operand
//   as they lie.  Softmax per column in 32-bit, base 2, the running maximum and sum kept by the column's four lanes.
// SPLITV (groups of at most 16 columns: single tokens): all four wavefronts compute the same scores and each takes
// a quarter of the value channels, so a lone token's workgroup still uses its four matrix units.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define TK 32                   // keys in a tile
#define VT_PITCH 40             // elements between the channels of the transposed values (80 bytes)
#define TILES_MAX_BLOCKS 2048   // page ids of a workgroup's key range that it keeps in LDS

template <int NKF, int NVT, bool SPLITV>
__global__ __launch_bounds__(256) void sink_attention_tiles_kernel(SinkArgs a, const int32_t* __restrict__ group_first,
                                                                   const int32_t* __restrict__ group_count,
                                                                   int head_block, int head_blocks) {
    constexpr int KD = NKF * 32, KP = KD + 8, CPK = NKF * 4;          // padded key channels, row pitch, 16-byte chunks a key
    constexpr int NSK = (TK * CPK + 255) / 256;                        // chunks of key rows a thread stages
    constexpr int CPV = NVT * 2, NSV = (TK * CPV + 255) / 256;         // the same for value rows of their own
    constexpr int NACC = SPLITV ? NVT / 4 : NVT;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    __bf16* k_lds = reinterpret_cast<__bf16*>(lds_raw);               // [TK][KP]
    __bf16* vt_lds = k_lds + TK * KP;                                  // [NVT * 16][VT_PITCH]
    int32_t* page_lds = reinterpret_cast<int32_t*>(vt_lds + NVT * 16 * VT_PITCH);      // [TILES_MAX_BLOCKS]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int group = blockIdx.x, kvh = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
    const int first = group_first[group], count = group_count[group];
    const int hg = a.q_heads / a.kv_heads;
    const int D = a.key_dim, V = a.value_dim;
    const bool shared_rows = a.v_pages == a.k_pages;
    const int p0 = a.positions[first], slot = a.slots[first];
    int kbegin = first_seen(p0, a.mask_kind, a.mask_size), kend = p0 + count;
    if (a.partial != nullptr) {                // this workgroup's share of the keys, from the group's first tile on
        const int base = (kbegin / TK) * TK + (int)blockIdx.z * a.split_keys;
        kbegin = max(kbegin, base);
        kend = min(kend, base + a.split_keys);
    }
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;

    // this lane's column
    const int col = (SPLITV ? 0 : wave * 16) + (lane & 15), b = lane >> 4;
    const int ti = col / head_block, hi = hb * head_block + col % head_block;
    const bool col_ok = ti < count && hi < hg;
    const int head = kvh * hg + (hi < hg ? hi : 0);
    const int m = first + (ti < count ? ti : 0);
    const int qpos = p0 + ti;
    const int qlo = first_seen(qpos, a.mask_kind, a.mask_size);
    const int last_lo = first_seen(p0 + count - 1, a.mask_kind, a.mask_size);      // (no token's range starts later)
    bf16x8 qf[NKF];
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int kf = 0; kf < NKF; ++kf) {
        const int d = kf * 32 + b * 8;
        qf[kf] = (col_ok && d < D) ? *reinterpret_cast<const bf16x8*>(a.q + (size_t)m * a.q_stride + (size_t)head * D + d) : zero8;
    }
    floatx4 acc[NACC];
#pragma unroll
    for (int j = 0; j < NACC; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
    float run_max = -INFINITY, run_sum = 0.f;
    const float scale2 = a.scale * 1.4426950408889634f;

    // the page ids of the workgroup's key range, once
    const int block0 = kbegin / a.page_size;
    const int n_blocks = kend > kbegin ? min((kend - 1) / a.page_size - block0 + 1, TILES_MAX_BLOCKS) : 0;
    for (int i = tid; i < n_blocks; i += 256) page_lds[i] = block0 + i < a.max_blocks ? table[block0 + i] : -1;
    __syncthreads();

    // A thread stages the same key of every tile (key = thread % 32: 256 is a multiple of it) and the chunks
    // thread / 32 + 8 i of its row: one row address a tile, then loads that do not wait for each other (addresses
    // are clamped and what must not count is zeroed afterwards: a load behind a branch would wait for the one before).
    bf16x8 kreg_a[NSK], vreg_a[NSV];
    const int my_key = tid & 31, my_chunk = tid >> 5;
    auto fetch = [&](int t0, bf16x8 (&kreg)[NSK], bf16x8 (&vreg)[NSV]) {
        const int kp = t0 + my_key;
        const bool inside = kp >= kbegin && kp < kend;
        const int blk = inside ? kp / a.page_size - block0 : 0;
        const int page = (inside && blk < n_blocks) ? page_lds[blk] : -1;
        const bool have = page >= 0;
        const long long r = have ? ((long long)page * a.kv_heads + kvh) * a.page_size + kp % a.page_size : 0;
        const __bf16* krow = a.k_pages + r * a.k_row;
#pragma unroll
        for (int i = 0; i < NSK; ++i) {
            const int d = (my_chunk + 8 * i) * 8;
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(krow + min(d, D - 8));
            kreg[i] = (have && d < D) ? v : zero8;
        }
        if (!shared_rows) {
            const __bf16* vrow = a.v_pages + r * a.v_row;
#pragma unroll
            for (int i = 0; i < NSV; ++i) {
                const int d = (my_chunk + 8 * i) * 8;
                const bf16x8 v = *reinterpret_cast<const bf16x8*>(vrow + min(d, V - 8));
                vreg[i] = (have && d < V) ? v : zero8;
            }
        }
    };
    // The transposed values go to LDS two keys a write: neighbouring lanes hold neighbouring keys, so a lane takes its
    // neighbour's 16-bit halves by a lane exchange (no LDS traffic) and writes the pair (key, key + 1) of a channel as
    // ONE 32-bit word -- the even lane the even channels, the odd lane the odd ones: half the LDS instructions of
    // eight 16-bit writes, which were what a tile of wide values waited for.
    const bool odd_key = my_key & 1;
    const int key_pair = my_key & ~1;
    auto transposed = [&](const bf16x8& rows, int d) {
        typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
        const u32x4 w = __builtin_bit_cast(u32x4, rows);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t own = w[c];
            const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)own, 0xB1, 0xF, 0xF, true);   // lane ^ 1
            const uint32_t pair = odd_key ? ((other >> 16) | (own & 0xffff0000u)) : ((own & 0xffffu) | (other << 16));
            const int channel = d + 2 * c + (odd_key ? 1 : 0);
            *reinterpret_cast<uint32_t*>(&vt_lds[channel * VT_PITCH + key_pair]) = channel < V ? pair : 0u;
        }
    };
    auto stage = [&](const bf16x8 (&kreg)[NSK], const bf16x8 (&vreg)[NSV]) {
#pragma unroll
        for (int i = 0; i < NSK; ++i) {
            const int d = (my_chunk + 8 * i) * 8;
            if (d < KD) {
                *reinterpret_cast<bf16x8*>(&k_lds[my_key * KP + d]) = kreg[i];
                if (shared_rows && d < NVT * 16) transposed(kreg[i], d);
            }
        }
        if (!shared_rows) {
#pragma unroll
            for (int i = 0; i < NSV; ++i) {
                const int d = (my_chunk + 8 * i) * 8;
                if (d < NVT * 16) transposed(vreg[i], d);
            }
        }
    };

    auto tile = [&](int t0) {
        // scores of this lane's column against the tile's keys 8 b .. 8 b + 7
        floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
        const int i16 = lane & 15;
        const int krow0 = 8 * (i16 >> 2) + (i16 & 3);
#pragma unroll
        for (int kf = 0; kf < NKF; ++kf) {
            const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(&k_lds[krow0 * KP + kf * 32 + b * 8]);
            const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(&k_lds[(krow0 + 4) * KP + kf * 32 + b * 8]);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[kf], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qf[kf], s1, 0, 0, 0);
        }
        float sc[8];
        float tile_max = -INFINITY;
        // a tile that every token of the group sees whole needs no comparisons (the same in every thread)
        const bool whole = t0 >= last_lo && t0 + TK - 1 <= p0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int kp = t0 + 8 * b + e;
            const float raw = e < 4 ? s0[e] : s1[e - 4];
            const bool seen = col_ok && (whole || (kp >= qlo && kp <= qpos));
            sc[e] = seen ? raw * scale2 : -INFINITY;
            tile_max = fmaxf(tile_max, sc[e]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, MLR_WAVE));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, MLR_WAVE));
        const float new_max = fmaxf(run_max, tile_max);
        // (the raw exponential instruction: its arguments are at most 0, and what underflows may be 0)
        const float corr = new_max > -INFINITY ? __builtin_amdgcn_exp2f(run_max - new_max) : 1.f;
        float part = 0.f;
        bf16x8 pf;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float p = new_max > -INFINITY ? __builtin_amdgcn_exp2f(sc[e] - new_max) : 0.f;
            part += p;
            pf[e] = (__bf16)p;
        }
        part += __shfl_xor(part, 16, MLR_WAVE);
        part += __shfl_xor(part, 32, MLR_WAVE);
        run_sum = run_sum * corr + part;
        run_max = new_max;
        // the sums so far are only scaled where some column's maximum rose (the same in every lane of the wavefront)
        const bool rose = __builtin_amdgcn_ballot_w64(corr != 1.f) != 0;
#pragma unroll
        for (int j = 0; j < NACC; ++j) {
            const int vt = SPLITV ? j * 4 + wave : j;
            if (vt * 16 < V) {                     // (the same in every lane)
                if (rose) acc[j] *= corr;
                const bf16x8 av = *reinterpret_cast<const bf16x8*>(&vt_lds[(vt * 16 + i16) * VT_PITCH + 8 * b]);
                acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, pf, acc[j], 0, 0, 0);
            }
        }
    };
    // The next tile's rows are asked for before this tile's products, unconditionally (beyond the range the rows come
    // out as zeros): a load behind a branch would make the loop wait for it where the branches join, before the
    // products it is meant to hide behind.
    const int t_first = (kbegin / TK) * TK;
    fetch(t_first, kreg_a, vreg_a);
    for (int t0 = t_first; t0 < kend; t0 += TK) {
        stage(kreg_a, vreg_a);
        __syncthreads();
        fetch(t0 + TK, kreg_a, vreg_a);
        tile(t0);
        __syncthreads();
    }
    if (a.partial != nullptr) {                // this range's share: the merge kernel finishes the column
        if (!col_ok) return;
        float* dst = a.partial + ((((size_t)group * a.group_tokens + ti) * a.q_heads + head) * a.splits + blockIdx.z) * (V + 4);
#pragma unroll
        for (int j = 0; j < NACC; ++j) {
            const int vt = SPLITV ? j * 4 + wave : j;
            if (vt * 16 < V) *reinterpret_cast<float4*>(dst + vt * 16 + 4 * b) = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
        }
        if (b == 0 && (!SPLITV || wave == 0)) {
            dst[V] = run_max;
            dst[V + 1] = run_sum;
        }
        return;
    }
    // the sink, and the division
    float top = run_max, den = run_sum, f = 1.f;
    if (a.sink != nullptr) {
        const float sk = a.sink[head] * 1.4426950408889634f;
        top = fmaxf(run_max, sk);
        f = run_max > -INFINITY ? exp2f(run_max - top) : 0.f;
        den = run_sum * f + exp2f(sk - top);
    }
    f = den > 0.f ? f / den : 0.f;
    if (!col_ok) return;
    __bf16* dst = a.out + (size_t)m * a.out_stride + (size_t)head * V;
#pragma unroll
    for (int j = 0; j < NACC; ++j) {
        const int vt = SPLITV ? j * 4 + wave : j;
        if (vt * 16 < V) {
            // accumulator element r of a lane: channel vt * 16 + 4 b + r of column lane % 16
            alignas(8) __bf16 four[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) four[r] = (__bf16)(acc[j][r] * f);
            *reinterpret_cast<uint2*>(dst + vt * 16 + 4 * b) = *reinterpret_cast<const uint2*>(four);
        }
    }
}

// The merge of the key ranges' shares (maxima and sums in the base-2 domain, as the kernel above leaves them), the
// sink and the division: one wavefront per (token of a group, head).
__global__ __launch_bounds__(64) void sink_tiles_combine_kernel(SinkArgs a, const int32_t* __restrict__ group_first,
                                                                const int32_t* __restrict__ group_count) {
    const int group = blockIdx.x, ti = blockIdx.z, head = blockIdx.y, lane = threadIdx.x;
    if (ti >= group_count[group]) return;
    const int m = group_first[group] + ti, V = a.value_dim;
    const float* base = a.partial + (((size_t)group * a.group_tokens + ti) * a.q_heads + head) * a.splits * (V + 4);
    float top = a.sink != nullptr ? a.sink[head] * 1.4426950408889634f : -INFINITY;
    const float sink2 = top;
    for (int z = 0; z < a.splits; ++z) top = fmaxf(top, base[(size_t)z * (V + 4) + V]);
    float den = a.sink != nullptr ? exp2f(sink2 - top) : 0.f;
    float num[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) num[i] = 0.f;
    for (int z = 0; z < a.splits; ++z) {
        const float* p = base + (size_t)z * (V + 4);
        const float zmax = p[V];
        if (!(zmax > -INFINITY)) continue;     // (a range beyond the token's keys)
        const float w = exp2f(zmax - top);
        den += w * p[V + 1];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = lane + 64 * i;
            if (c < V) num[i] += w * p[c];
        }
    }
    const float inv = den > 0.f ? 1.0f / den : 0.f;
    __bf16* dst = a.out + (size_t)m * a.out_stride + (size_t)head * V;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int c = lane + 64 * i;
        if (c < V) dst[c] = (__bf16)(num[i] * inv);
    }
}

template <int NKF, int NVT, bool SPLITV>
static int launch_sink_tiles(const SinkArgs& a, const int32_t* first, const int32_t* count, int groups, int head_block,
                             int head_blocks, hipStream_t stream) {
    const size_t lds = ((size_t)TK * (NKF * 32 + 8) + (size_t)NVT * 16 * VT_PITCH) * sizeof(__bf16) +
                       TILES_MAX_BLOCKS * sizeof(int32_t);
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(&sink_attention_tiles_kernel<NKF, NVT, SPLITV>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
            return -3;
        raised = true;
    }
    sink_attention_tiles_kernel<NKF, NVT, SPLITV><<<dim3(groups, a.kv_heads * head_blocks, a.partial ? a.splits : 1), 256, lds,
                                                   stream>>>(a, first, count, head_block, head_blocks);
    if (a.partial != nullptr)
        sink_tiles_combine_kernel<<<dim3(groups, a.q_heads, a.group_tokens), 64, 0, stream>>>(a, first, count);
    return (int)hipGetLastError();
}
#endif

extern "C" {

int mlr_sink_attention(const void* q, long q_stride, const void* k_pages, long k_row, const void* v_pages, long v_row,
                       const int32_t* block_table, int max_blocks, const int32_t* slots, const int32_t* positions,
                       const float* sink, void* out, long out_stride, int rows, int q_heads, int kv_heads, int key_dim,
                       int value_dim, int page_size, int mask_kind, int mask_size, float scale, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (key_dim > MAX_KEY_DIM || value_dim > 64 * MAX_V_REGS || q_heads > 65535 || kv_heads <= 0 ||
        q_heads % kv_heads != 0 || (mask_kind != MASK_ALL && mask_size <= 0))
        return -1;
    SinkArgs a{(const elem_t*)q, q_stride, (const elem_t*)k_pages, k_row, (const elem_t*)v_pages, v_row, block_table,
               slots, positions, sink, (elem_t*)out, out_stride, max_blocks, q_heads, kv_heads, key_dim, value_dim,
               page_size, mask_kind, mask_size, scale, nullptr, 0, 1, 1};
    sink_attention_kernel<<<dim3(rows, q_heads), 64, 0, stream>>>(a);
    return (int)hipGetLastError();
}

int mlr_sink_qkv_prep(const void* proj, long ld, const float* bias, void* q_out, void* k_pages, long k_row,
                      void* v_pages, long v_row, const int32_t* block_table, int max_blocks, const int32_t* slots,
                      const int32_t* positions, const float* q_norm_w, const float* k_norm_w, float eps,
                      const float* rope, int rot_dim, int rows, int q_heads, int kv_heads, int key_dim, int value_dim,
                      int page_size, int write_cache, int norm_mode, int interleaved, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (key_dim > MAX_KEY_DIM || q_heads + 2 * kv_heads > 65535 || rot_dim > key_dim || (rot_dim & 1) || norm_mode < 0 ||
        norm_mode > 2)
        return -1;
    sink_qkv_prep_kernel<<<dim3(rows, q_heads + 2 * kv_heads), 64, 0, stream>>>(
        (const elem_t*)proj, ld, bias, (elem_t*)q_out, (elem_t*)k_pages, k_row, (elem_t*)v_pages, v_row, block_table,
        max_blocks, slots, positions, q_norm_w, k_norm_w, eps, rope, rot_dim, q_heads, kv_heads, key_dim, value_dim,
        page_size, write_cache, norm_mode, interleaved);
    return (int)hipGetLastError();
}

int mlr_latent_prep(const void* q_src, long q_ld, const void* kv_src, long kv_ld, void* q_out, void* pages, long row_width,
                    const int32_t* block_table, int max_blocks, const int32_t* slots, const int32_t* positions,
                    const float* norm_w, float eps, const float* rope, int rows, int heads, int dim, int rot, int rank,
                    int page_size, int write_cache, int interleaved, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (heads + 1 > 65535 || (rot & 1) || rot <= 0 || rope == nullptr) return -1;
    latent_prep_kernel<<<dim3(rows, heads + 1), 64, 0, stream>>>(
        (const elem_t*)q_src, q_ld, (const elem_t*)kv_src, kv_ld, (elem_t*)q_out, (elem_t*)pages, row_width, block_table,
        max_blocks, slots, positions, norm_w, eps, rope, heads, dim, rot, rank, page_size, write_cache, interleaved);
    return (int)hipGetLastError();
}

// The matrix-core kernel over `groups` groups of consecutive tokens of one request each (group_first / group_count:
// device vectors), every group holding at most 64 / head_block tokens (16 / head_block with split_values, which
// deals the value channels out to the four wavefronts: single tokens).  head_block: a power of two, query heads of
// one kv head side by side in a workgroup's columns.  max_context: the longest context of the step (what a
// workgroup walks at most when no mask bounds it).  splits > 1: a group's keys in `splits` ranges of split_keys keys
// (a multiple of 32) from its first tile on, one workgroup each, their shares in `partial` (floats: groups x tokens a
// group x q_heads x splits x (value_dim + 4)) merged by a second launch.  Returns 1 when the sizes are not this
// kernel's.
int mlr_sink_attention_tiles(const void* q, long q_stride, const void* k_pages, long k_row, const void* v_pages,
                             long v_row, const int32_t* block_table, int max_blocks, const int32_t* slots,
                             const int32_t* positions, const float* sink, void* out, long out_stride,
                             const int32_t* group_first, const int32_t* group_count, int groups, int head_block,
                             int split_values, int q_heads, int kv_heads, int key_dim, int value_dim, int page_size,
                             int mask_kind, int mask_size, int max_context, float scale, float* partial, int split_keys,
                             int splits, hipStream_t stream) {
#if MLR_BF16
    if (groups <= 0) return 0;
    {
        // the keys that one workgroup may have to walk: its page ids must fit what it keeps of them
        const long reach = mask_kind == MASK_ALL ? (long)max_context : (long)mask_size + 64;
        if (reach / page_size + 2 > TILES_MAX_BLOCKS) return 1;
    }
    if (key_dim % 8 != 0 || value_dim % 16 != 0 || key_dim > 576 || value_dim > 512 || k_row % 8 != 0 || v_row % 8 != 0 ||
        q_stride % 8 != 0 || out_stride % 4 != 0 || kv_heads <= 0 || q_heads % kv_heads != 0)
        return 1;
    if (head_block < 1 || head_block > (split_values ? 16 : 64) || (head_block & (head_block - 1)) != 0 ||
        (mask_kind != MASK_ALL && mask_size <= 0))
        return -1;
    const int hg = q_heads / kv_heads, head_blocks = (hg + head_block - 1) / head_block;
    if ((long)kv_heads * head_blocks > 65535) return -2;
    SinkArgs a{(const elem_t*)q, q_stride, (const elem_t*)k_pages, k_row, (const elem_t*)v_pages, v_row, block_table,
               slots, positions, sink, (elem_t*)out, out_stride, max_blocks, q_heads, kv_heads, key_dim, value_dim,
               page_size, mask_kind, mask_size, scale, splits > 1 ? partial : nullptr, split_keys, splits > 1 ? splits : 1,
               (split_values ? 16 : 64) / head_block};
    if (splits > 1 && (partial == nullptr || split_keys <= 0 || split_keys % TK != 0 || splits > 65535 || a.group_tokens > 65535))
        return -1;
    const int nkf = (key_dim + 31) / 32, nvt = value_dim / 16;
#define MLR_SINK_CLASS(NKF, NVT)                                                                                       \
    if (nkf <= NKF && nvt <= NVT)                                                                                      \
        return split_values ? launch_sink_tiles<NKF, NVT, true>(a, group_first, group_count, groups, head_block,      \
                                                                 head_blocks, stream)                                  \
                            : launch_sink_tiles<NKF, NVT, false>(a, group_first, group_count, groups, head_block,     \
                                                                  head_blocks, stream);
    MLR_SINK_CLASS(2, 4)
    MLR_SINK_CLASS(4, 8)
    MLR_SINK_CLASS(8, 16)
    MLR_SINK_CLASS(18, 32)
#undef MLR_SINK_CLASS
    return 1;
#else
    return 1;
#endif
}

}  // extern "C"
