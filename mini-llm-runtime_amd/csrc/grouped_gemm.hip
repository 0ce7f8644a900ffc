// Products of many small matrices in one launch, and the routing of a mixture of experts around them.
//
// `grouped_gemm`: out_g[r, n] = act(sum_k a_g[r, k] * w_g[n, k]) for every group g, w_g = w + g * w_group being
// [N, K] row-major.  Two ways of saying which rows a group has:
//   offsets == null: every group takes the rows 0 .. M - 1, group g reading a + g * a_group and writing
//     out + g * out_group with row strides lda / ldo: one projection per head on slices of wider rows;
//   offsets != null: group g takes the rows offsets[g] .. offsets[g + 1] - 1 of a list sorted by group (rows of
//     out; a's row is gather[row] when gather != null): the experts of a routed feed-forward.
// act: none, or relu(x)^2.  Every output element is one sum over k in ascending order whatever rows lie beside
// it, so a row's result does not depend on the batch.  Accumulation is 32-bit; the bfloat16 engine multiplies on
// the matrix cores (v_mfma_f32_16x16x32_bf16, operands staged through LDS), the float engine with plain FMAs.
//
// Routing (32-bit): `router_topk_kernel` (sigmoid of a token's router logits, the best groups of neighbouring
// experts, the best experts within them), `route_sort_kernel` (the chosen (token, expert) pairs
// sorted by expert: offsets, the token of every sorted row, the sorted row of every pair),
// `route_combine_kernel` (a token's output: the weighted sum of its experts' rows, in the order of its choices).
#include "common.h"

#define ACT_NONE 0
#define ACT_RELU2 1
// (bfloat16 kernels) gated forms: the weight holds a gate's and its up projection's rows in turn, 16 of the one and the
// matching 16 of the other ([gate 0..15 | up 0..15 | gate 16..31 | ...]); out[m, f] = act(gate_f) * up_f, N / 2 columns
#define ACT_GATED_SILU 2
#define ACT_GATED_GELU_TANH 3

struct GroupedArgs {
    const elem_t* a; long lda; long a_group;
    const elem_t* w; long w_group;
    void* out; long ldo; long out_group;
    const int32_t* offsets; const int32_t* gather;
    int M, N, K, groups, act, out_float;
};

#define GBM 64              // rows and columns of the small workgroup tile (the float engine's only one)
#define GBN 64

// Which group and which rows this workgroup serves: (group, first row, one beyond the group's last row), or
// group < 0 when the launch has more workgroups than the groups have tiles.
__device__ __forceinline__ void tile_of(const GroupedArgs& g, int& group, int& row0, int& row_end, const int tile_rows = GBM) {
    if (g.offsets == nullptr) {
        group = blockIdx.z;
        row0 = blockIdx.y * tile_rows;
        row_end = g.M;
        return;
    }
    int tile = blockIdx.y;
    group = -1;
    for (int e = 0; e < g.groups; ++e) {
        const int first = g.offsets[e], count = g.offsets[e + 1] - first;
        const int tiles = (count + tile_rows - 1) / tile_rows;
        if (tile < tiles) {
            group = e;
            row0 = first + tile * tile_rows;
            row_end = first + count;
            return;
        }
        tile -= tiles;
    }
}

__device__ __forceinline__ float activate(float x, int act) {
    if (act == ACT_RELU2) {
        const float r = fmaxf(x, 0.f);
        return r * r;
    }
    return x;
}

__device__ __forceinline__ float gate_act(float g, int act) {
    if (act == ACT_GATED_SILU) return g / (1.0f + expf(-g));
    return 0.5f * g * (1.0f + tanhf(0.79788456080286535588f * (g + 0.044715f * g * g * g)));
}

#if !MLR_BF16
#define GBK 16
__global__ __launch_bounds__(256) void grouped_gemm_kernel(GroupedArgs g) {
    __shared__ float as[GBK][GBM + 4];
    __shared__ float ws[GBK][GBN + 4];
    int group, m0, m_end;
    tile_of(g, group, m0, m_end);
    if (group < 0 || m0 >= m_end) return;
    const int t = threadIdx.x, n0 = blockIdx.x * GBN;
    const int tx = t % 16, ty = t / 16;
    const int lrow = t / 4, lk = (t % 4) * 4;
    const float* a = g.a + (g.offsets ? 0 : (size_t)group * g.a_group);
    const float* w = g.w + (size_t)group * g.w_group;
    float* out = (float*)g.out + (g.offsets ? 0 : (size_t)group * g.out_group);
    long arow = -1;                            // the row of a that this thread stages
    if (m0 + lrow < m_end) arow = g.gather ? g.gather[m0 + lrow] : m0 + lrow;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < g.K; k0 += GBK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e, wn = n0 + lrow;
            as[lk + e][lrow] = (arow >= 0 && k < g.K) ? a[arow * g.lda + k] : 0.f;
            ws[lk + e][lrow] = (wn < g.N && k < g.K) ? w[(size_t)wn * g.K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GBK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = as[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= m_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < g.N) out[(size_t)m * g.ldo + n] = activate(acc[i][j], g.act);
        }
    }
}
#else
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
__device__ __forceinline__ bf16x8 load_k8(const __bf16* p, int k, int K, bool vector_ok) {
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (vector_ok && k + 8 <= K) {
        v = *reinterpret_cast<const bf16x8*>(p + k);
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (k + e < K) v[e] = p[k + e];
    }
    return v;
}

// A workgroup of 2 x 2 wavefronts, each T x T tiles of 16 x 16: T = 2 owns 64 x 64 outputs and takes k in blocks of
// 128, T = 4 owns 128 x 128 (half the operand traffic an output: for many rows) in blocks of 64.  A block is staged
// through LDS, the next block on its way from memory into registers meanwhile (a block's loads are all asked for
// before anything waits).  Rows of a staged block lie 16 bytes further apart than their data, so that the 16-byte
// reads of 16 rows meet no bank twice.
template <int T>
__global__ __launch_bounds__(256) void grouped_gemm_kernel(GroupedArgs g) {
    constexpr int BM = 32 * T, BN = 32 * T, BK = T == 2 ? 128 : 64, PITCH = BK + 8;
    constexpr int RT = 256 / BM;                     // threads that share a row of a staged operand
    constexpr int CH = BK / 8 / RT;                  // 16-byte chunks of it that one thread stages
    __shared__ __attribute__((aligned(16))) __bf16 as[BM * PITCH];
    __shared__ __attribute__((aligned(16))) __bf16 ws[BN * PITCH];
    int group, m0, m_end;
    tile_of(g, group, m0, m_end, BM);
    if (group < 0 || m0 >= m_end) return;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, n0 = blockIdx.x * BN;
    const int wm = wave >> 1, wn = wave & 1;
    const __bf16* a = g.a + (g.offsets ? 0 : (size_t)group * g.a_group);
    const __bf16* w = g.w + (size_t)group * g.w_group;
    const size_t out_base = g.offsets ? 0 : (size_t)group * g.out_group;
    // 16-byte loads where every row starts at a multiple of 16 bytes
    const bool a_vec = (g.K % 8) == 0 && (g.lda % 8) == 0 && (g.a_group % 8) == 0 &&
                       (reinterpret_cast<uintptr_t>(g.a) % 16) == 0;
    const bool w_vec = (g.K % 8) == 0 && (g.w_group % 8) == 0 && (reinterpret_cast<uintptr_t>(g.w) % 16) == 0;
    const int srow = t / RT, sk = (t % RT) * 8;      // this thread stages row srow of both operands: chunks sk + 8 RT c
    long arow = -1;
    if (m0 + srow < m_end) arow = g.gather ? g.gather[m0 + srow] : m0 + srow;
    const bool wrow_ok = n0 + srow < g.N;
    const __bf16* ap = a + (arow >= 0 ? arow : 0) * g.lda;
    const __bf16* wp = w + (size_t)(wrow_ok ? n0 + srow : 0) * g.K;
    floatx4 acc[T][T];
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int j = 0; j < T; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 ar[CH], wr[CH];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k = k0 + sk + 8 * RT * c;
            ar[c] = load_k8(ap, k, g.K, a_vec);
            wr[c] = load_k8(wp, k, g.K, w_vec);
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < g.K; k0 += BK) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            *reinterpret_cast<bf16x8*>(&as[srow * PITCH + sk + 8 * RT * c]) = arow >= 0 ? ar[c] : zero;
            *reinterpret_cast<bf16x8*>(&ws[srow * PITCH + sk + 8 * RT * c]) = wrow_ok ? wr[c] : zero;
        }
        __syncthreads();
        if (k0 + BK < g.K) fetch(k0 + BK);
        const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 32) {
            bf16x8 af[T], wf[T];
#pragma unroll
            for (int i = 0; i < T; ++i)
                af[i] = *reinterpret_cast<const bf16x8*>(&as[((wm * T + i) * 16 + frag_row) * PITCH + kk + frag_k]);
#pragma unroll
            for (int j = 0; j < T; ++j)
                wf[j] = *reinterpret_cast<const bf16x8*>(&ws[((wn * T + j) * 16 + frag_row) * PITCH + kk + frag_k]);
#pragma unroll
            for (int i = 0; i < T; ++i)
#pragma unroll
                for (int j = 0; j < T; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
    // accumulator element r of a lane: row (lane / 16) * 4 + r, column lane % 16
    if (g.act >= ACT_GATED_SILU) {
        // a wavefront's neighbouring column tiles hold a gate block and its up block: half as many columns leave
#pragma unroll
        for (int i = 0; i < T; ++i) {
#pragma unroll
            for (int j = 0; j < T; j += 2) {
                if (n0 + (wn * T + j) * 16 + (lane & 15) >= g.N) continue;
                const int n = (n0 >> 1) + ((wn * T + j) >> 1) * 16 + (lane & 15);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int m = m0 + (wm * T + i) * 16 + (lane >> 4) * 4 + r;
                    if (m >= m_end) continue;
                    const float y = gate_act(acc[i][j][r], g.act) * acc[i][j + 1][r];
                    const size_t at = out_base + (size_t)m * g.ldo + n;
                    if (g.out_float) ((float*)g.out)[at] = y;
                    else ((__bf16*)g.out)[at] = (__bf16)y;
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
#pragma unroll
        for (int j = 0; j < T; ++j) {
            const int n = n0 + (wn * T + j) * 16 + (lane & 15);
            if (n >= g.N) continue;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + (wm * T + i) * 16 + (lane >> 4) * 4 + r;
                if (m >= m_end) continue;
                const float y = activate(acc[i][j][r], g.act);
                const size_t at = out_base + (size_t)m * g.ldo + n;
                if (g.out_float) ((float*)g.out)[at] = y;
                else ((__bf16*)g.out)[at] = (__bf16)y;
            }
        }
    }
}
#endif

// ---------------------------------------------------------------------------------------------------------
#define MAX_EXPERTS 256         // 64 lanes x EXPERT_REGS
#define EXPERT_REGS 4

// The largest value among the lanes' candidates and, among equals, the lowest index; every lane gets both.
__device__ __forceinline__ void wave_best(float& value, int& index) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(value, off, MLR_WAVE);
        const int oi = __shfl_xor(index, off, MLR_WAVE);
        if (ov > value || (ov == value && oi < index)) {
            value = ov;
            index = oi;
        }
    }
}

// One wavefront a token.  s = sigmoid(z), z[m] the token's router logits (float: a product of the framework's own,
// 32-bit sums).  The experts form `group_count`
// equal groups of neighbours; a group's score is the sum of its two largest s (of its only one, when a group is
// one expert); only experts of the `group_keep` best groups stand; of those the `top` largest s are chosen
// (ties: the lower index), ids[m][i] in descending order of s with weights[m][i] = s itself.
// With `correction` [experts] the choice (of groups and of experts) goes by s + correction while the weights stay
// the plain s; with `renorm` the chosen weights are divided by their sum (+ 1e-20); `out_scale` multiplies them.
__global__ __launch_bounds__(64) void router_topk_kernel(const float* __restrict__ z, int32_t* __restrict__ ids,
                                                         float* __restrict__ weights, int experts, int top,
                                                         int group_count, int group_keep,
                                                         const float* __restrict__ correction, int renorm, float out_scale) {
    __shared__ float s_lds[MAX_EXPERTS];      // what the choice goes by
    __shared__ float w_lds[MAX_EXPERTS];      // the plain scores
    __shared__ float g_lds[MAX_EXPERTS];
    const int m = blockIdx.x, lane = threadIdx.x;
    for (int e = lane; e < experts; e += 64) {
        const float sc = 1.0f / (1.0f + expf(-z[(size_t)m * experts + e]));
        w_lds[e] = sc;
        s_lds[e] = correction != nullptr ? sc + correction[e] : sc;
    }
    __syncthreads();
    const int per = experts / group_count;
    for (int gidx = lane; gidx < group_count; gidx += 64) {
        float first = -INFINITY, second = -INFINITY;
        for (int i = 0; i < per; ++i) {
            const float v = s_lds[gidx * per + i];
            if (v > first) {
                second = first;
                first = v;
            } else if (v > second) {
                second = v;
            }
        }
        g_lds[gidx] = per >= 2 ? first + second : first;
    }
    __syncthreads();
    // the groups that stand: group_keep times the best of those left; their experts become candidates
    float cand[EXPERT_REGS];
#pragma unroll
    for (int i = 0; i < EXPERT_REGS; ++i) cand[i] = -INFINITY;
    for (int round = 0; round < group_keep; ++round) {
        float best = -INFINITY;
        int which = 0x7fffffff;
        for (int gidx = lane; gidx < group_count; gidx += 64) {
            const float v = g_lds[gidx];
            if (v > best) {                    // (ascending indices: the lowest among equals stays)
                best = v;
                which = gidx;
            }
        }
        wave_best(best, which);
        if (which == 0x7fffffff) break;
        __syncthreads();
        if (lane == 0) g_lds[which] = -INFINITY;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < EXPERT_REGS; ++i) {
            const int e = lane + 64 * i;
            if (e < experts && e / per == which) cand[i] = s_lds[e];
        }
    }
    float chosen_sum = 0.f;
    for (int round = 0; round < top; ++round) {
        float best = -INFINITY;
        int which = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < EXPERT_REGS; ++i) {
            const int e = lane + 64 * i;
            if (e < experts && cand[i] > best) {
                best = cand[i];
                which = e;
            }
        }
        wave_best(best, which);
        if (which == 0x7fffffff) which = 0, best = 0.f;      // (fewer candidates than `top`: refused on the host)
#pragma unroll
        for (int i = 0; i < EXPERT_REGS; ++i)
            if (lane + 64 * i == which) cand[i] = -INFINITY;
        chosen_sum += w_lds[which];                           // (the same on every lane, in the order of the choices)
        if (lane == 0) {
            ids[(size_t)m * top + round] = which;
            weights[(size_t)m * top + round] = w_lds[which];
        }
    }
    if (renorm || out_scale != 1.0f) {
        __syncthreads();
        for (int r = lane; r < top; r += 64) {
            float w = weights[(size_t)m * top + r];
            if (renorm) w = w / (chosen_sum + 1e-20f);
            weights[(size_t)m * top + r] = w * out_scale;
        }
    }
}

// The `pairs` chosen (token, expert) pairs sorted by expert, by ONE workgroup: offsets[e] .. offsets[e + 1] are
// expert e's rows of the sorted list, token_of[row] the pair's token, row_of[pair] where the pair went.  The
// order of an expert's rows among themselves is whatever the atomics give; no result depends on it.
__global__ __launch_bounds__(1024) void route_sort_kernel(const int32_t* __restrict__ ids, int pairs, int top,
                                                          int experts, int32_t* __restrict__ offsets,
                                                          int32_t* __restrict__ token_of, int32_t* __restrict__ row_of) {
    __shared__ int count[MAX_EXPERTS + 1];
    __shared__ int cursor[MAX_EXPERTS];
    const int t = threadIdx.x;
    for (int e = t; e <= experts; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int i = t; i < pairs; i += blockDim.x) atomicAdd(&count[ids[i]], 1);
    __syncthreads();
    if (t == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            const int n = count[e];
            cursor[e] = at;
            offsets[e] = at;
            at += n;
        }
        offsets[experts] = at;
    }
    __syncthreads();
    for (int i = t; i < pairs; i += blockDim.x) {
        const int row = atomicAdd(&cursor[ids[i]], 1);
        token_of[row] = i / top;
        row_of[i] = row;
    }
}

// out[m, :] = sum_i weights[m][i] * y[row_of[m * top + i], :], the sum in 32-bit in the order of the choices.
__global__ void route_combine_kernel(const elem_t* __restrict__ y, const int32_t* __restrict__ row_of,
                                     const float* __restrict__ weights, elem_t* __restrict__ out, int width, int top) {
    const int m = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float sum = 0.f;
        for (int i = 0; i < top; ++i)
            sum = fmaf(weights[(size_t)m * top + i], to_float(y[(size_t)row_of[(size_t)m * top + i] * width + c]), sum);
        out[(size_t)m * width + c] = from_float<elem_t>(sum);
    }
}

extern "C" {

int mlr_grouped_gemm(const void* a, long lda, long a_group, const void* w, long w_group, void* out, long ldo,
                     long out_group, const int32_t* offsets, const int32_t* gather, int M, int N, int K, int groups,
                     int act, int out_float, hipStream_t stream) {
    if (M <= 0 || N <= 0 || groups <= 0) return 0;
    if (K <= 0 || act < ACT_NONE || act > ACT_GATED_GELU_TANH) return -1;
#if !MLR_BF16
    if (act >= ACT_GATED_SILU) return -3;            // (the gated forms are the matrix-core kernels')
    out_float = 1;
#else
    if (act >= ACT_GATED_SILU && N % 32 != 0) return -3;
#endif
    GroupedArgs g{(const elem_t*)a, lda, a_group, (const elem_t*)w, w_group, out, ldo, out_group, offsets, gather,
                  M, N, K, groups, act, out_float};
#if MLR_BF16
    // experts with many rows each: the large tile (310 -> 340 TFLOP/s at 2048 tokens of width 2048, 390 -> 420 at width
    // 4096; the products a head, with inner sizes of 128 to 512, are faster on the small one)
    if (offsets != nullptr && (long)M >= 256L * groups && N >= 128) {
        const int row_tiles = (M + 127) / 128 + (offsets ? groups : 0);
        if (row_tiles > 65535 || groups > 65535) return -2;
        grouped_gemm_kernel<4><<<dim3((N + 127) / 128, row_tiles, offsets ? 1 : groups), 256, 0, stream>>>(g);
        return (int)hipGetLastError();
    }
#endif
    const int row_tiles = (M + GBM - 1) / GBM + (offsets ? groups : 0);
    if (row_tiles > 65535 || groups > 65535) return -2;
    dim3 grid((N + GBN - 1) / GBN, row_tiles, offsets ? 1 : groups);
#if MLR_BF16
    grouped_gemm_kernel<2><<<grid, 256, 0, stream>>>(g);
#else
    grouped_gemm_kernel<<<grid, 256, 0, stream>>>(g);
#endif
    return (int)hipGetLastError();
}

int mlr_router_topk(const float* z, int32_t* ids, float* weights, int rows, int experts, int top, int group_count,
                    int group_keep, const float* correction, int renorm, float out_scale, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (experts < 1 || experts > MAX_EXPERTS || group_count < 1 || experts % group_count != 0 || group_keep < 1 ||
        group_keep > group_count || top < 1 || top > group_keep * (experts / group_count))
        return -1;
    router_topk_kernel<<<rows, 64, 0, stream>>>(z, ids, weights, experts, top, group_count, group_keep, correction, renorm,
                                                out_scale);
    return (int)hipGetLastError();
}

int mlr_route_sort(const int32_t* ids, int pairs, int top, int experts, int32_t* offsets, int32_t* token_of,
                   int32_t* row_of, hipStream_t stream) {
    if (pairs <= 0) return 0;
    if (experts < 1 || experts > MAX_EXPERTS || top < 1) return -1;
    route_sort_kernel<<<1, 1024, 0, stream>>>(ids, pairs, top, experts, offsets, token_of, row_of);
    return (int)hipGetLastError();
}

int mlr_route_combine(const void* y, const int32_t* row_of, const float* weights, void* out, int rows, int width,
                      int top, hipStream_t stream) {
    if (rows <= 0) return 0;
    route_combine_kernel<<<rows, 256, 0, stream>>>((const elem_t*)y, row_of, weights, (elem_t*)out, width, top);
    return (int)hipGetLastError();
}

}  // extern "C"
