// Mixers with a state of fixed size per request: a short causal convolution over channels, the decays of
// gated linear attention and of Mamba-2, and the linear recurrence both share,
//     S_t = diag(a_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t        (S: N key channels x V value channels),
// run token by token in 32-bit from the state that earlier steps left.  A step brings any mix of prompt
// portions and single tokens; a request's tokens are consecutive rows of the batch (`seg_first`, `seg_count`,
// one entry a request of the step).  The live state of a request is read from `live + slot * stride`, the
// state that the step leads to is written to `stage + slot * stride` (the engine makes it live when every
// layer has run).  Every sum is taken in an order that depends on the token's own data only, so a token's
// result does not depend on how its request was cut into steps or on what else the batch holds.
//
// The delta rule (`delta_rule_kernel`) is the same walk with a write that first takes back what the state already
// holds for the token's key:  S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t.
//
// Long portions (the bfloat16 engine) run the recurrence over pieces of a request side by side, in three passes:
// every piece from a zero state, leaving its last state L_c and the product A_c of its decays; then, piece after
// piece, the state each piece starts from, S_(c+1) = diag(A_c) S_c + L_c (element by element, from the live
// state); then every piece again from its S_c, writing the outputs.  Twice the arithmetic, as many workgroups as
// pieces; the result differs from the token-by-token order by 32-bit rounding only.
#include "common.h"

__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---- short causal convolution -----------------------------------------------------------------------
// out[r, c] = act(b[c] + sum_j w[c, j] * in(r, taps - 1 - j)) with in(r, d) the channel's input d tokens before
// row r: a row of this step when the request brought it, else the request's state, which holds its last
// taps - 1 inputs, oldest first, as [taps - 1][C] floats (zeros at a sequence's start).  The last row of a
// request in the step writes the state that follows.  One thread per (row, channel).
struct ConvArgs {
    const elem_t* x; long x_stride;
    const float* w; const float* b;
    elem_t* out; long out_stride;
    const float* live; float* stage; long state_stride;
    const int32_t* slots; const int32_t* positions;
    int rows, channels, taps, silu, write_state;
};

#define CONV_MAX_TAPS 8

__global__ __launch_bounds__(256) void causal_conv_kernel(ConvArgs a) {
    const int r = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    const int slot = a.slots[r], pos = a.positions[r];
    const int before = a.taps - 1;
    int have = 0;                              // rows right before r that are this request's previous tokens
    while (have < before && r - have - 1 >= 0 && a.slots[r - have - 1] == slot && a.positions[r - have - 1] == pos - have - 1) ++have;
    const bool last = r + 1 >= a.rows || a.slots[r + 1] != slot || a.positions[r + 1] != pos + 1;
    if (c >= a.channels) return;
    float in[CONV_MAX_TAPS];                   // in[d]: the input d tokens back
#pragma unroll
    for (int d = 0; d < CONV_MAX_TAPS; ++d) {
        if (d > before) { in[d] = 0.f; continue; }
        if (d <= have) in[d] = to_float(a.x[(size_t)(r - d) * a.x_stride + c]);
        else in[d] = a.live[(size_t)slot * a.state_stride + (size_t)(before - d + have) * a.channels + c];
    }
    float acc = a.b ? a.b[c] : 0.f;
#pragma unroll
    for (int d = CONV_MAX_TAPS - 1; d >= 0; --d) {         // oldest input first; tap j = taps - 1 - d
        if (d <= before) acc += a.w[(size_t)c * a.taps + (before - d)] * in[d];
    }
    if (a.silu) acc = acc / (1.0f + expf(-acc));
    a.out[(size_t)r * a.out_stride + c] = from_float<elem_t>(acc);
    if (last && a.write_state) {
#pragma unroll
        for (int d = 0; d < CONV_MAX_TAPS - 1; ++d) {
            if (d < before) a.stage[(size_t)slot * a.state_stride + (size_t)(before - 1 - d) * a.channels + c] = in[d];
        }
    }
}

// ---- decays ---------------------------------------------------------------------------------------------
// Gated linear attention: the logarithm of alpha = sigmoid(z + b)^(1 / tau), that is -softplus(-(z + b)) / tau.
__global__ void gla_log_decay_kernel(const elem_t* __restrict__ z, const float* __restrict__ bias, float* __restrict__ out,
                                     size_t rows, int width, float inv_tau) {
    const size_t total = rows * width;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const float x = to_float(z[i]) + (bias ? bias[i % width] : 0.f);
        out[i] = -softplus_f(-x) * inv_tau;
    }
}

// Mamba-2: the step size dt = softplus(raw + dt_bias[h]) (no clamp) and the log decay -exp(A_log[h]) * dt.
__global__ void mamba_step_kernel(const elem_t* __restrict__ raw, long raw_stride, const float* __restrict__ dt_bias,
                                  const float* __restrict__ a_log, float* __restrict__ dt, float* __restrict__ log_decay,
                                  size_t rows, int heads) {
    const size_t total = rows * heads;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / heads;
        const int h = (int)(i % heads);
        const float step = softplus_f(to_float(raw[r * raw_stride + h]) + dt_bias[h]);
        dt[i] = step;
        log_decay[i] = -expf(a_log[h]) * step;
    }
}

// ---- the recurrence --------------------------------------------------------------------------------------
struct ScanArgs {
    const elem_t* q; long q_stride;            // q[r * q_stride + (head / heads_per_group) * N + i]
    const elem_t* k; long k_stride;
    const elem_t* v; long v_stride;            // v[r * v_stride + head * V + j]
    const float* log_decay; long decay_stride; // per channel: [r * stride + head * N + i]; else [r * stride + head]
    const float* v_scale; long v_scale_stride; // factor on v, [r * stride + head], or null
    const float* skip;                         // out += skip[head] * v (unscaled), or null
    float* out;                                // [rows, heads * V]
    const float* live; float* stage; long state_stride;     // a request's S as [heads][N][V]
    const int32_t* seg_first; const int32_t* seg_count; const int32_t* slots;
    int heads, heads_per_group, N, V, decay_per_channel, write_state;
    float q_scale;
    int silu;                                  // q, k and v pass silu as they are read (before the factors)
    float* piece_state;                        // [pieces][heads][N][V]: L_c after the first pass, S_c after the second
    float* piece_decay;                        // [pieces][heads][N]: A_c
};

#define SCAN_COLS 64
#define SCAN_PARTS 4

// One workgroup per (request of the step, head, 64 value channels): wavefront p holds rows [p NR, (p + 1) NR)
// of S for its 64 columns in registers, a lane a column.  Tokens are staged TILE at a time through LDS
// (decays exponentiated, q scaled, v scaled); after a tile the four partial sums of o are added in the order
// of the parts.
// MODE 0: a request's rows of the step from its live state to the staged one.  MODE 1: a piece from a zero state,
// no outputs; leaves L_c and A_c.  MODE 2: a piece from S_c, outputs only.  (In modes 1 and 2 `seg_first` and
// `seg_count` name the pieces.)
template <int NR, int TILE, int MODE>
__global__ __launch_bounds__(256) void linear_recurrence_kernel(ScanArgs a) {
    constexpr int NPAD = NR * SCAN_PARTS;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* a_lds = lds;                                   // [TILE][NPAD]
    float* k_lds = a_lds + TILE * NPAD;
    float* q_lds = k_lds + TILE * NPAD;
    float* v_lds = q_lds + TILE * NPAD;                   // [TILE][COLS]
    float* o_lds = v_lds + TILE * SCAN_COLS;              // [PARTS][TILE][COLS]
    const int seg = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * SCAN_COLS;
    const int r0 = a.seg_first[seg], n = a.seg_count[seg];
    const int slot = a.slots[r0];
    const int j = threadIdx.x & 63, part = threadIdx.x >> 6;
    const int col = col0 + j;
    const int N = a.N, V = a.V;
    const int qk_head = head / a.heads_per_group;
    const size_t state_at = (size_t)slot * a.state_stride + (size_t)head * N * V;
    const size_t piece_at = ((size_t)seg * a.heads + head) * N * V;
    float S[NR], A[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int i = part * NR + r;
        const bool in = i < N && col < V;
        S[r] = MODE == 1 || !in ? 0.f : MODE == 0 ? a.live[state_at + (size_t)i * V + col] : a.piece_state[piece_at + (size_t)i * V + col];
        A[r] = 1.f;
    }
    for (int t0 = 0; t0 < n; t0 += TILE) {
        const int nt = min(TILE, n - t0);
        __syncthreads();                                  // the tile before is read and written out
        for (int idx = threadIdx.x; idx < nt * NPAD; idx += 256) {
            const int t = idx / NPAD, i = idx % NPAD;
            const size_t row = (size_t)(r0 + t0 + t);
            float da = 0.f, dk = 0.f, dq = 0.f;
            if (i < N) {
                da = expf(a.log_decay[row * a.decay_stride + (a.decay_per_channel ? head * N + i : head)]);
                dk = to_float(a.k[row * a.k_stride + qk_head * N + i]);
                dq = to_float(a.q[row * a.q_stride + qk_head * N + i]);
                if (a.silu) { dk = silu_f(dk); dq = silu_f(dq); }
                dq *= a.q_scale;
            }
            a_lds[idx] = da; k_lds[idx] = dk; q_lds[idx] = dq;
        }
        for (int idx = threadIdx.x; idx < nt * SCAN_COLS; idx += 256) {
            const int t = idx / SCAN_COLS, c = col0 + idx % SCAN_COLS;
            const size_t row = (size_t)(r0 + t0 + t);
            float x = 0.f;
            if (c < V) {
                x = to_float(a.v[row * a.v_stride + head * V + c]);
                if (a.silu) x = silu_f(x);
                if (a.v_scale) x *= a.v_scale[row * a.v_scale_stride + head];
            }
            v_lds[idx] = x;
        }
        __syncthreads();
        for (int t = 0; t < nt; ++t) {
            const float x = v_lds[t * SCAN_COLS + j];
            const float* at = a_lds + t * NPAD + part * NR;
            const float* kt = k_lds + t * NPAD + part * NR;
            const float* qt = q_lds + t * NPAD + part * NR;
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                S[r] = at[r] * S[r] + kt[r] * x;
                if (MODE == 1) A[r] *= at[r];
                else o += qt[r] * S[r];
            }
            if (MODE != 1) o_lds[(part * TILE + t) * SCAN_COLS + j] = o;
        }
        if (MODE == 1) continue;
        __syncthreads();
        for (int idx = threadIdx.x; idx < nt * SCAN_COLS; idx += 256) {
            const int t = idx / SCAN_COLS, c = col0 + idx % SCAN_COLS;
            if (c >= V) continue;
            const size_t row = (size_t)(r0 + t0 + t);
            float o = o_lds[idx];
#pragma unroll
            for (int p = 1; p < SCAN_PARTS; ++p) o += o_lds[p * TILE * SCAN_COLS + idx];
            if (a.skip) {
                const float x = to_float(a.v[row * a.v_stride + head * V + c]);
                o += a.skip[head] * (a.silu ? silu_f(x) : x);
            }
            a.out[row * ((size_t)a.heads * V) + head * V + c] = o;
        }
    }
    if (MODE == 0 && a.write_state && col < V) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int i = part * NR + r;
            if (i < N) a.stage[state_at + (size_t)i * V + col] = S[r];
        }
    }
    if (MODE == 1) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int i = part * NR + r;
            if (i < N && col < V) a.piece_state[piece_at + (size_t)i * V + col] = S[r];
            if (i < N && col == 0) a.piece_decay[((size_t)seg * a.heads + head) * N + i] = A[r];
        }
    }
}

// The second pass: one thread per element (head, i, j) of the state walks the pieces in their order.  A piece
// whose request differs from the piece before starts from that request's live state; where a request's pieces
// end its state is staged.  piece_state[c] holds L_c on entry and S_c, the state piece c starts from, on exit.
__global__ void piece_states_kernel(ScanArgs a, int pieces) {
    const size_t per = (size_t)a.heads * a.N * a.V;
    const size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= per) return;
    const size_t hi = e / a.V;                 // head * N + i
    float S = 0.f;
    for (int c = 0; c < pieces; ++c) {
        const int slot = a.slots[a.seg_first[c]];
        if (c == 0 || a.slots[a.seg_first[c - 1]] != slot) S = a.live[(size_t)slot * a.state_stride + e];
        const float last = a.piece_state[(size_t)c * per + e];
        a.piece_state[(size_t)c * per + e] = S;
        S = a.piece_decay[(size_t)c * a.heads * a.N + hi] * S + last;
        if (a.write_state && (c + 1 == pieces || a.slots[a.seg_first[c + 1]] != slot)) a.stage[(size_t)slot * a.state_stride + e] = S;
    }
}

// ---- the delta rule ----------------------------------------------------------------------------------------
// Decays of the key channels from a step size per channel: log g = -exp(A_log[head]) * softplus(z + bias), z the
// 32-bit output of a low-rank pair of projections laid out [heads][N].
__global__ void channel_log_decay_kernel(const float* __restrict__ z, const float* __restrict__ bias,
                                         const float* __restrict__ a_log, float* __restrict__ out, size_t rows, int width,
                                         int per_head) {
    const size_t total = rows * width;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int c = (int)(i % width);
        out[i] = -expf(a_log[c / per_head]) * softplus_f(z[i] + (bias ? bias[c] : 0.f));
    }
}

struct DeltaArgs {
    const elem_t* q; long q_stride;            // q[r * q_stride + (head / heads_per_group) * N + i], as projected
    const elem_t* k; long k_stride;
    const elem_t* v; long v_stride;            // v[r * v_stride + head * V + j]
    const float* log_decay;                    // [rows][heads * N], or with decay_per_head [rows][heads]
    const float* beta_raw; long beta_stride;   // beta = sigmoid(beta_raw[r * stride + head])
    float* out;                                // [rows, heads * V]
    const float* live; float* stage; long state_stride;     // a request's S as [heads][N][V]
    const int32_t* seg_first; const int32_t* seg_count; const int32_t* slots;
    int heads, heads_per_group, N, V, write_state, unit_norm;
    float q_scale, unit_eps;
    int decay_per_head;                        // one decay for all key channels of a head
};

// Where the log decay of (row, head, key channel i) lies.
__device__ __forceinline__ size_t decay_at(const DeltaArgs& a, size_t row, int head, int i) {
    return a.decay_per_head ? row * (size_t)a.heads + head : row * ((size_t)a.heads * a.N) + (size_t)head * a.N + i;
}

#define DELTA_TILE 16

// One wavefront per (request of the step, head, COLS value channels), COLS = 64 / PARTS: lane (part, column) holds
// rows [part NR, (part + 1) NR) of its column of S in registers.  Tokens are staged DELTA_TILE at a time through LDS:
// q and k made unit vectors over the head's N channels (x / sqrt(sum x^2 + unit_eps); q times q_scale), the decays
// exponentiated, beta = sigmoid(raw), k . q of every token.  A token then costs one pass over the lane's rows for
// (g S)^T k and (g S)^T q, an exchange between the parts, and one pass for the write; the read-out after the write is
// o = (g S)^T q + (k . q) u.  Every sum's order follows from the head's sizes alone.
template <int NR, int PARTS>
__global__ __launch_bounds__(64) void delta_rule_kernel(DeltaArgs a) {
    constexpr int COLS = 64 / PARTS;
    constexpr int NPAD = NR * PARTS;
    __shared__ __attribute__((aligned(16))) float g_lds[DELTA_TILE * NPAD];
    __shared__ __attribute__((aligned(16))) float k_lds[DELTA_TILE * NPAD];
    __shared__ __attribute__((aligned(16))) float q_lds[DELTA_TILE * NPAD];
    __shared__ float v_lds[DELTA_TILE * COLS];
    __shared__ float beta_lds[DELTA_TILE], kq_lds[DELTA_TILE];
    const int seg = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * COLS;
    const int r0 = a.seg_first[seg], n = a.seg_count[seg];
    const int slot = a.slots[r0];
    const int lane = threadIdx.x, j = lane % COLS, part = lane / COLS;
    const int col = col0 + j;
    const int N = a.N, V = a.V;
    const int qk_head = head / a.heads_per_group;
    const size_t state_at = (size_t)slot * a.state_stride + (size_t)head * N * V;
    float S[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        const int i = part * NR + r;
        S[r] = i < N && col < V ? a.live[state_at + (size_t)i * V + col] : 0.f;
    }
    for (int t0 = 0; t0 < n; t0 += DELTA_TILE) {
        const int nt = min(DELTA_TILE, n - t0);
        __syncthreads();                                  // the tile before has been read
        for (int t = 0; t < nt; ++t) {
            const size_t row = (size_t)(r0 + t0 + t);
            float qq = 0.f, kk = 0.f;
            for (int i = lane; i < NPAD; i += 64) {
                float dq = 0.f, dk = 0.f, dg = 0.f;
                if (i < N) {
                    dq = to_float(a.q[row * a.q_stride + qk_head * N + i]);
                    dk = to_float(a.k[row * a.k_stride + qk_head * N + i]);
                    dg = expf(a.log_decay[decay_at(a, row, head, i)]);
                }
                qq += dq * dq;
                kk += dk * dk;
                q_lds[t * NPAD + i] = dq; k_lds[t * NPAD + i] = dk; g_lds[t * NPAD + i] = dg;
            }
            float fq = a.q_scale, fk = 1.0f;
            if (a.unit_norm) {
                fq = a.q_scale / sqrtf(wave_sum(qq) + a.unit_eps);
                fk = 1.0f / sqrtf(wave_sum(kk) + a.unit_eps);
            }
            float dot = 0.f;
            for (int i = lane; i < NPAD; i += 64) {      // (each lane returns to the channels it wrote)
                const float dq = q_lds[t * NPAD + i] * fq, dk = k_lds[t * NPAD + i] * fk;
                q_lds[t * NPAD + i] = dq; k_lds[t * NPAD + i] = dk;
                dot += dq * dk;
            }
            dot = wave_sum(dot);
            if (lane == 0) {
                kq_lds[t] = dot;
                beta_lds[t] = sigmoid_f(a.beta_raw[row * a.beta_stride + head]);
            }
        }
        for (int idx = lane; idx < nt * COLS; idx += 64) {
            const int t = idx / COLS, c = col0 + idx % COLS;
            v_lds[idx] = c < V ? to_float(a.v[(size_t)(r0 + t0 + t) * a.v_stride + head * V + c]) : 0.f;
        }
        __syncthreads();
        for (int t = 0; t < nt; ++t) {
            const float* gt = g_lds + t * NPAD + part * NR;
            const float* kt = k_lds + t * NPAD + part * NR;
            const float* qt = q_lds + t * NPAD + part * NR;
            float sk = 0.f, sq = 0.f;
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                S[r] *= gt[r];
                sk += kt[r] * S[r];
                sq += qt[r] * S[r];
            }
#pragma unroll
            for (int off = COLS; off < 64; off <<= 1) {   // the parts of a column lie COLS lanes apart
                sk += __shfl_xor(sk, off, 64);
                sq += __shfl_xor(sq, off, 64);
            }
            const float u = beta_lds[t] * (v_lds[t * COLS + j] - sk);
#pragma unroll
            for (int r = 0; r < NR; ++r) S[r] += kt[r] * u;
            if (part == 0 && col < V) a.out[(size_t)(r0 + t0 + t) * ((size_t)a.heads * V) + head * V + col] = sq + kq_lds[t] * u;
        }
    }
    if (a.write_state && col < V) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const int i = part * NR + r;
            if (i < N) a.stage[state_at + (size_t)i * V + col] = S[r];
        }
    }
}


// ---- the delta rule over chunks of tokens --------------------------------------------------------------------
// A request's rows are cut into chunks of at most DC tokens.  With c_t[i] the sum of a chunk's log decays of key
// channel i up to and including token t, and S0 the state the chunk starts from, the rule's writes u_t obey
//     u_t = beta_t (v_t - S0^T (k_t e^{c_t}) - sum_{s<t} (sum_i k_t[i] k_s[i] e^{c_t[i] - c_s[i]}) u_s),
// a unit lower-triangular system (I + A) U = beta (V - Khat S0) whose inverse T depends on the chunk's keys, decays
// and beta alone.  The first kernel (one workgroup per chunk and head, all side by side) leaves in scratch memory
//     W = T (beta Khat) [DC, N],  Y = T (beta V) [DC, V],  B[t, s] = sum_i q_t[i] k_s[i] e^{c_t[i] - c_s[i]} (s <= t),
//     Qhat[t] = q_t e^{c_t},  Kbar[s] = k_s e^{c_last - c_s},  G = e^{c_last};
// the second (one workgroup per request, head and 16 or 32 value channels) walks a request's chunks in
// their order with the state in LDS:  U = Y - W S0;  O = Qhat S0 + B U;  S <- diag(G) S0 + Kbar^T U.
// Every exponent is a difference c_t - c_s with s <= t or c_t itself, so nothing overflows however strong a decay
// is.  The result differs from the token-by-token kernel's by 32-bit rounding.
#define DELTA_CHUNK 32

struct DeltaChunkArgs {
    DeltaArgs d;
    const int32_t* chunk_first; const int32_t* chunk_count;     // the chunks, a request's one after the other
    float* scratch;                                              // [chunks][heads][delta_chunk_floats(N, V)]
};

__host__ __device__ inline size_t delta_chunk_floats(int N, int V) {
    return (size_t)DELTA_CHUNK * (3 * N + V + DELTA_CHUNK) + N;
}

__global__ __launch_bounds__(256) void delta_chunk_prepare_kernel(DeltaChunkArgs g) {
    constexpr int C = DELTA_CHUNK, CS = DELTA_CHUNK + 1;
    const DeltaArgs& a = g.d;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int N = a.N, V = a.V, NS = N + 1;
    float* q_l = lds;                    // [C][NS]
    float* k_l = q_l + C * NS;
    float* c_l = k_l + C * NS;
    float* A_l = c_l + C * NS;           // [C][CS]
    float* B_l = A_l + C * CS;
    float* T_l = B_l + C * CS;
    float* beta_l = T_l + C * CS;        // [C]
    const int chunk = blockIdx.x, head = blockIdx.y;
    const int r0 = g.chunk_first[chunk], n = g.chunk_count[chunk];
    const int qk_head = head / a.heads_per_group;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float* base = g.scratch + ((size_t)chunk * a.heads + head) * delta_chunk_floats(N, V);
    float* W = base;
    float* Qh = W + (size_t)C * N;
    float* Kb = Qh + (size_t)C * N;
    float* Y = Kb + (size_t)C * N;
    float* B = Y + (size_t)C * V;
    float* G = B + C * C;
    for (int idx = tid; idx < C * N; idx += 256) {
        const int t = idx / N, i = idx % N;
        float dq = 0.f, dk = 0.f, dc = 0.f;
        if (t < n) {
            const size_t row = (size_t)(r0 + t);
            dq = to_float(a.q[row * a.q_stride + qk_head * N + i]);
            dk = to_float(a.k[row * a.k_stride + qk_head * N + i]);
            dc = a.log_decay[decay_at(a, row, head, i)];
        }
        q_l[t * NS + i] = dq; k_l[t * NS + i] = dk; c_l[t * NS + i] = dc;
    }
    __syncthreads();
    for (int t = wave; t < C; t += 4) {                     // unit vectors, q scaled; beta
        float qq = 0.f, kk = 0.f;
        for (int i = lane; i < N; i += 64) {
            const float dq = q_l[t * NS + i], dk = k_l[t * NS + i];
            qq += dq * dq;
            kk += dk * dk;
        }
        float fq = a.q_scale, fk = 1.0f;
        if (a.unit_norm) {
            fq = a.q_scale / sqrtf(wave_sum(qq) + a.unit_eps);
            fk = 1.0f / sqrtf(wave_sum(kk) + a.unit_eps);
        }
        for (int i = lane; i < N; i += 64) { q_l[t * NS + i] *= fq; k_l[t * NS + i] *= fk; }
        if (lane == 0) beta_l[t] = t < n ? sigmoid_f(a.beta_raw[(size_t)(r0 + t) * a.beta_stride + head]) : 0.f;
    }
    for (int i = tid; i < N; i += 256) {                    // c_t: the running sum of the log decays (rows past n add 0)
        float sum = 0.f;
        for (int t = 0; t < C; ++t) { sum += c_l[t * NS + i]; c_l[t * NS + i] = sum; }
    }
    __syncthreads();
    for (int p = tid; p < C * C; p += 256) {
        const int t = p / C, s = p % C;
        float sa = 0.f, sb = 0.f;
        if (s <= t && t < n) {
            const float* ct = c_l + t * NS; const float* cs = c_l + s * NS;
            const float* kt = k_l + t * NS; const float* ks = k_l + s * NS; const float* qt = q_l + t * NS;
            for (int i = 0; i < N; ++i) {
                const float x = ks[i] * expf(ct[i] - cs[i]);
                sa += kt[i] * x;
                sb += qt[i] * x;
            }
        }
        A_l[t * CS + s] = s < t ? beta_l[t] * sa : 0.f;
        B_l[t * CS + s] = sb;
        B[t * C + s] = sb;
    }
    for (int idx = tid; idx < C * N; idx += 256) {          // Qhat, Kbar, G (they read what the loop above reads)
        const int t = idx / N, i = idx % N;
        const float ct = c_l[t * NS + i], last = c_l[(C - 1) * NS + i];
        Qh[idx] = q_l[t * NS + i] * expf(ct);
        Kb[idx] = k_l[t * NS + i] * expf(last - ct);
        if (t == 0) G[i] = expf(last);
    }
    __syncthreads();
    if (tid < C) {                                          // T = (I + A)^-1, a column a lane, row after row
        const int j = tid;
        for (int t = 0; t < C; ++t) {
            float x = t == j ? 1.f : 0.f;
            for (int s = 0; s < t; ++s) x -= A_l[t * CS + s] * T_l[s * CS + j];
            T_l[t * CS + j] = x;
        }
    }
    for (int idx = tid; idx < C * N; idx += 256) {          // beta Khat in q's place
        const int t = idx / N, i = idx % N;
        q_l[t * NS + i] = beta_l[t] * k_l[t * NS + i] * expf(c_l[t * NS + i]);
    }
    __syncthreads();
    for (int idx = tid; idx < C * N; idx += 256) {
        const int t = idx / N, i = idx % N;
        float acc = 0.f;
        for (int s = 0; s <= t; ++s) acc += T_l[t * CS + s] * q_l[s * NS + i];
        W[idx] = acc;
    }
    for (int idx = tid; idx < C * V; idx += 256) {
        const int t = idx / V, j = idx % V;
        float acc = 0.f;
        const int last = min(t, n - 1);
        for (int s = 0; s <= last; ++s)
            acc += T_l[t * CS + s] * beta_l[s] * to_float(a.v[(size_t)(r0 + s) * a.v_stride + head * V + j]);
        Y[idx] = acc;
    }
}

template <int VEC> struct alignas(4 * VEC) DeltaVec { float v[VEC]; };

// VEC value channels a thread, 8 * VEC a workgroup: the narrower form fills the GPU when heads and value channels are few.
template <int VEC>
__global__ __launch_bounds__(256) void delta_chunk_scan_kernel(DeltaChunkArgs g) {
    constexpr int C = DELTA_CHUNK, CS = DELTA_CHUNK + 1, COLS = 8 * VEC;
    constexpr int PER = DELTA_CHUNK * 128 / 256;           // elements of a [C][N] tile a thread moves, N <= 128
    constexpr int PER_B = DELTA_CHUNK * DELTA_CHUNK / 256;
    typedef DeltaVec<VEC> vec_t;
    const DeltaArgs& a = g.d;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int N = a.N, V = a.V, NS = N + 1;
    float* S_l = lds;                    // [N][COLS]
    float* U_l = S_l + N * COLS;         // [C][COLS]
    float* W_l = U_l + C * COLS;         // [C][NS]: W, then Kbar
    float* Q_l = W_l + C * NS;           // [C][NS]: Qhat
    float* B_l = Q_l + C * NS;           // [C][CS]
    float* G_l = B_l + C * CS;           // [N]
    const int seg = blockIdx.x, head = blockIdx.y, col0 = blockIdx.z * COLS;
    const int r0 = a.seg_first[seg], n = a.seg_count[seg];
    const int slot = a.slots[r0];
    const int tid = threadIdx.x, t = tid >> 3, jq = (tid & 7) * VEC;
    int chunk0 = 0;
    for (int s = 0; s < seg; ++s) chunk0 += (a.seg_count[s] + C - 1) / C;
    const size_t per = delta_chunk_floats(N, V);
    const size_t state_at = (size_t)slot * a.state_stride + (size_t)head * N * V;
    const int tile = C * N;
    int at_lds[PER];                                        // where this thread's tile elements go in LDS
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        const int idx = tid + 256 * r;
        at_lds[r] = (idx / N) * NS + idx % N;
    }
    for (int idx = tid; idx < N * COLS; idx += 256) {
        const int i = idx / COLS, c = col0 + idx % COLS;
        S_l[idx] = c < V ? a.live[state_at + (size_t)i * V + c] : 0.f;
    }
    // a chunk's W, Qhat, B, G and Y are on their way into registers while the chunk before is worked on; Kbar while
    // the chunk's own first products run
    float w_next[PER], q_next[PER], k_next[PER], b_next[PER_B], y_next[VEC], g_next;
    const float* base = g.scratch + ((size_t)chunk0 * a.heads + head) * per;
    auto fetch = [&](const float* from) {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int idx = tid + 256 * r;
            w_next[r] = idx < tile ? from[idx] : 0.f;
            q_next[r] = idx < tile ? from[tile + idx] : 0.f;
        }
        const float* Y = from + 3 * (size_t)tile;
        const float* B = Y + (size_t)C * V;
#pragma unroll
        for (int e = 0; e < VEC; ++e) y_next[e] = col0 + jq + e < V ? Y[(size_t)t * V + col0 + jq + e] : 0.f;
#pragma unroll
        for (int r = 0; r < PER_B; ++r) b_next[r] = B[tid + 256 * r];
        g_next = tid < N ? B[C * C + tid] : 0.f;
    };
    fetch(base);
    for (int c0 = 0; c0 < n; c0 += C) {
        const int nt = min(C, n - c0);
        const float* Kb = base + 2 * (size_t)tile;
        __syncthreads();                                    // the state is whole, the tiles of the chunk before are read
#pragma unroll
        for (int r = 0; r < PER; ++r)
            if (tid + 256 * r < tile) { W_l[at_lds[r]] = w_next[r]; Q_l[at_lds[r]] = q_next[r]; }
#pragma unroll
        for (int r = 0; r < PER_B; ++r) B_l[((tid + 256 * r) / C) * CS + (tid + 256 * r) % C] = b_next[r];
        if (tid < N) G_l[tid] = g_next;
        float u[VEC], o[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) { u[e] = y_next[e]; o[e] = 0.f; }
#pragma unroll
        for (int r = 0; r < PER; ++r) k_next[r] = tid + 256 * r < tile ? Kb[tid + 256 * r] : 0.f;
        __syncthreads();
        {
            const float* wt = W_l + t * NS;
            const float* qt = Q_l + t * NS;
#pragma unroll 8
            for (int i = 0; i < N; ++i) {
                const float w = wt[i], qv = qt[i];
                const vec_t s4 = *reinterpret_cast<const vec_t*>(S_l + i * COLS + jq);
#pragma unroll
                for (int e = 0; e < VEC; ++e) { u[e] -= w * s4.v[e]; o[e] += qv * s4.v[e]; }
            }
        }
        {
            vec_t u4;
#pragma unroll
            for (int e = 0; e < VEC; ++e) u4.v[e] = u[e];
            *reinterpret_cast<vec_t*>(U_l + t * COLS + jq) = u4;
        }
        __syncthreads();                                    // U is whole; W's tile has been read
#pragma unroll
        for (int r = 0; r < PER; ++r)
            if (tid + 256 * r < tile) W_l[at_lds[r]] = k_next[r];
        if (c0 + C < n) {
            base += (size_t)a.heads * per;
            fetch(base);
        }
        {
            const float* bt = B_l + t * CS;
#pragma unroll 4
            for (int s = 0; s <= t; ++s) {
                const float w = bt[s];
                const vec_t u4 = *reinterpret_cast<const vec_t*>(U_l + s * COLS + jq);
#pragma unroll
                for (int e = 0; e < VEC; ++e) o[e] += w * u4.v[e];
            }
        }
        if (t < nt) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (col0 + jq + e < V) a.out[(size_t)(r0 + c0 + t) * ((size_t)a.heads * V) + head * V + col0 + jq + e] = o[e];
        }
        __syncthreads();                                    // Kbar is in W's place
        for (int i = t; i < N; i += C) {                   // (a thread's own elements of S: no other thread reads them now)
            vec_t s4 = *reinterpret_cast<const vec_t*>(S_l + i * COLS + jq);
            const float gi = G_l[i];
#pragma unroll
            for (int e = 0; e < VEC; ++e) s4.v[e] *= gi;
#pragma unroll 8
            for (int s = 0; s < C; ++s) {
                const float w = W_l[s * NS + i];
                const vec_t u4 = *reinterpret_cast<const vec_t*>(U_l + s * COLS + jq);
#pragma unroll
                for (int e = 0; e < VEC; ++e) s4.v[e] += w * u4.v[e];
            }
            *reinterpret_cast<vec_t*>(S_l + i * COLS + jq) = s4;
        }
    }
    __syncthreads();
    if (a.write_state)
        for (int idx = tid; idx < N * COLS; idx += 256) {
            const int i = idx / COLS, c = col0 + idx % COLS;
            if (c < V) a.stage[state_at + (size_t)i * V + c] = S_l[idx];
        }
}

template <int NR, int PARTS>
static int launch_delta(const DeltaArgs& a, int segments, hipStream_t stream) {
    constexpr int COLS = 64 / PARTS;
    delta_rule_kernel<NR, PARTS><<<dim3(segments, a.heads, (a.V + COLS - 1) / COLS), 64, 0, stream>>>(a);
    return (int)hipGetLastError();
}

template <int NR, int TILE>
static int launch_scan(const ScanArgs& a, int segments, hipStream_t stream) {
    const size_t lds = sizeof(float) * ((size_t)3 * TILE * NR * SCAN_PARTS + (size_t)TILE * SCAN_COLS * (1 + SCAN_PARTS));
    dim3 grid(segments, a.heads, (a.V + SCAN_COLS - 1) / SCAN_COLS);
    if (a.piece_state == nullptr) {
        linear_recurrence_kernel<NR, TILE, 0><<<grid, 256, lds, stream>>>(a);
        return (int)hipGetLastError();
    }
    linear_recurrence_kernel<NR, TILE, 1><<<grid, 256, lds, stream>>>(a);
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    const size_t per = (size_t)a.heads * a.N * a.V;
    piece_states_kernel<<<(unsigned)((per + 255) / 256), 256, 0, stream>>>(a, segments);
    err = (int)hipGetLastError();
    if (err != 0) return err;
    linear_recurrence_kernel<NR, TILE, 2><<<grid, 256, lds, stream>>>(a);
    return (int)hipGetLastError();
}

static int grid_for(size_t count, int block) {
    size_t g = (count + block - 1) / block;
    return (int)(g > 65535 ? 65535 : (g == 0 ? 1 : g));
}

extern "C" {

int mlr_causal_conv(const void* x, long x_stride, const float* w, const float* b, void* out, long out_stride,
                    const float* live, float* stage, long state_stride, const int32_t* slots, const int32_t* positions,
                    int rows, int channels, int taps, int silu, int write_state, hipStream_t stream) {
    if (rows <= 0 || channels <= 0) return 0;
    if (taps < 1 || taps > CONV_MAX_TAPS) return -1;
    ConvArgs a{(const elem_t*)x, x_stride, w, b, (elem_t*)out, out_stride, live, stage, state_stride, slots, positions,
               rows, channels, taps, silu, write_state};
    causal_conv_kernel<<<dim3(rows, (channels + 255) / 256), 256, 0, stream>>>(a);
    return (int)hipGetLastError();
}

int mlr_gla_log_decay(const void* z, const float* bias, float* out, int rows, int width, float inv_tau, hipStream_t stream) {
    if (rows <= 0) return 0;
    gla_log_decay_kernel<<<grid_for((size_t)rows * width, 256), 256, 0, stream>>>((const elem_t*)z, bias, out, (size_t)rows,
                                                                                 width, inv_tau);
    return (int)hipGetLastError();
}

int mlr_mamba_step(const void* raw, long raw_stride, const float* dt_bias, const float* a_log, float* dt, float* log_decay,
                   int rows, int heads, hipStream_t stream) {
    if (rows <= 0) return 0;
    mamba_step_kernel<<<grid_for((size_t)rows * heads, 256), 256, 0, stream>>>((const elem_t*)raw, raw_stride, dt_bias, a_log,
                                                                              dt, log_decay, (size_t)rows, heads);
    return (int)hipGetLastError();
}

int mlr_linear_recurrence(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                          const float* log_decay, long decay_stride, int decay_per_channel, const float* v_scale,
                          long v_scale_stride, const float* skip, float q_scale, float* out, const float* live, float* stage,
                          long state_stride, const int32_t* seg_first, const int32_t* seg_count, const int32_t* slots,
                          int segments, int heads, int heads_per_group, int n_keys, int n_values, int write_state,
                          float* piece_state, float* piece_decay, int silu, hipStream_t stream) {
    // piece_state, piece_decay given: `seg_first`/`seg_count` name pieces of requests (a request's pieces one after
    // the other), run side by side in three passes; [segments][heads][n_keys][n_values] and [segments][heads][n_keys]
    if (segments <= 0) return 0;
    if (n_keys < 1 || n_keys > 256 || n_values < 1 || heads < 1 || heads_per_group < 1 || heads % heads_per_group) return -1;
    ScanArgs a{(const elem_t*)q, q_stride, (const elem_t*)k, k_stride, (const elem_t*)v, v_stride, log_decay, decay_stride,
               v_scale, v_scale_stride, skip, out, live, stage, state_stride, seg_first, seg_count, slots, heads,
               heads_per_group, n_keys, n_values, decay_per_channel, write_state, q_scale, silu, piece_state, piece_decay};
    if ((piece_state == nullptr) != (piece_decay == nullptr)) return -2;
    const int nr = (n_keys + SCAN_PARTS - 1) / SCAN_PARTS;
    if (nr <= 8) return launch_scan<8, 16>(a, segments, stream);
    if (nr <= 16) return launch_scan<16, 16>(a, segments, stream);
    if (nr <= 32) return launch_scan<32, 16>(a, segments, stream);
    return launch_scan<64, 8>(a, segments, stream);
}

int mlr_channel_log_decay(const float* z, const float* bias, const float* a_log, float* out, int rows, int heads, int n_keys,
                          hipStream_t stream) {
    if (rows <= 0) return 0;
    if (heads < 1 || n_keys < 1) return -1;
    channel_log_decay_kernel<<<grid_for((size_t)rows * heads * n_keys, 256), 256, 0, stream>>>(z, bias, a_log, out, (size_t)rows,
                                                                                            heads * n_keys, n_keys);
    return (int)hipGetLastError();
}

// The delta rule over the step's requests (seg_first, seg_count: one entry a request).  A lane keeps at most 64 rows of
// its column of S: up to 64 key channels a lane holds a whole column (64 columns a wavefront), up to 128 two lanes share
// one, up to 256 four; heads of few value channels use the narrower layouts too, so that their lanes are not idle.
int mlr_delta_rule(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                   const float* log_decay, const float* beta_raw, long beta_stride, float* out, const float* live, float* stage,
                   long state_stride, const int32_t* seg_first, const int32_t* seg_count, const int32_t* slots, int segments,
                   int heads, int heads_per_group, int n_keys, int n_values, int write_state, int unit_norm, float q_scale,
                   float unit_eps, int decay_per_head, hipStream_t stream) {
    if (segments <= 0) return 0;
    if (n_keys < 1 || n_keys > 256 || n_values < 1 || heads < 1 || heads > 65535 || heads_per_group < 1 ||
        heads % heads_per_group)
        return -1;
    DeltaArgs a{(const elem_t*)q, q_stride, (const elem_t*)k, k_stride, (const elem_t*)v, v_stride, log_decay, beta_raw,
                beta_stride, out, live, stage, state_stride, seg_first, seg_count, slots, heads, heads_per_group, n_keys,
                n_values, write_state, unit_norm, q_scale, unit_eps, decay_per_head};
    int parts = n_keys > 128 ? 4 : n_keys > 64 ? 2 : 1;
    if (n_values <= 16 && parts < 4) parts = 4;
    else if (n_values <= 32 && parts < 2) parts = 2;
    const int nr = (n_keys + parts - 1) / parts;
#define MLR_DELTA(PARTS)                                                        \
    if (parts == PARTS) {                                                       \
        if (nr <= 8) return launch_delta<8, PARTS>(a, segments, stream);        \
        if (nr <= 16) return launch_delta<16, PARTS>(a, segments, stream);      \
        if (nr <= 32) return launch_delta<32, PARTS>(a, segments, stream);      \
        return launch_delta<64, PARTS>(a, segments, stream);                    \
    }
    MLR_DELTA(1)
    MLR_DELTA(2)
    MLR_DELTA(4)
#undef MLR_DELTA
    return -1;
}

// The delta rule in chunks (see delta_chunk_prepare_kernel): `chunk_first`/`chunk_count` name the step's chunks of at
// most DELTA_CHUNK tokens, a request's chunks one after the other and the requests in the order of `seg_first`;
// scratch: chunks * heads * mlr_delta_chunk_floats(n_keys, n_values) floats.  Up to 128 key channels a head.
long mlr_delta_chunk_floats(int n_keys, int n_values) { return (long)delta_chunk_floats(n_keys, n_values); }
int mlr_delta_chunk_tokens() { return DELTA_CHUNK; }

int mlr_delta_rule_chunked(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride,
                           const float* log_decay, const float* beta_raw, long beta_stride, float* out, const float* live,
                           float* stage, long state_stride, const int32_t* seg_first, const int32_t* seg_count,
                           const int32_t* slots, int segments, const int32_t* chunk_first, const int32_t* chunk_count, int chunks,
                           float* scratch, int heads, int heads_per_group, int n_keys, int n_values, int write_state,
                           int unit_norm, float q_scale, float unit_eps, int decay_per_head, hipStream_t stream) {
    if (segments <= 0 || chunks <= 0) return 0;
    if (n_keys < 1 || n_keys > 128 || n_values < 1 || heads < 1 || heads > 65535 || heads_per_group < 1 ||
        heads % heads_per_group || scratch == nullptr)
        return -1;
    DeltaChunkArgs g{{(const elem_t*)q, q_stride, (const elem_t*)k, k_stride, (const elem_t*)v, v_stride, log_decay, beta_raw,
                      beta_stride, out, live, stage, state_stride, seg_first, seg_count, slots, heads, heads_per_group, n_keys,
                      n_values, write_state, unit_norm, q_scale, unit_eps, decay_per_head},
                     chunk_first, chunk_count, scratch};
    const int C = DELTA_CHUNK, NS = n_keys + 1;
    const size_t lds1 = sizeof(float) * ((size_t)3 * C * NS + (size_t)3 * C * (C + 1) + C);
    delta_chunk_prepare_kernel<<<dim3(chunks, heads), 256, lds1, stream>>>(g);
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    // 32 value channels a workgroup where that fills the GPU, else 16
    const bool wide = (long)segments * heads * ((n_values + 31) / 32) >= 256;
    const int cols = wide ? 32 : 16;
    const size_t lds2 = sizeof(float) * ((size_t)n_keys * cols + (size_t)C * cols + (size_t)2 * C * NS + (size_t)C * (C + 1) + n_keys);
    const dim3 grid(segments, heads, (n_values + cols - 1) / cols);
    if (wide) delta_chunk_scan_kernel<4><<<grid, 256, lds2, stream>>>(g);
    else delta_chunk_scan_kernel<2><<<grid, 256, lds2, stream>>>(g);
    return (int)hipGetLastError();
}

}  // extern "C"
