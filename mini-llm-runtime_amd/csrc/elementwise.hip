// Row-wise kernels of the decoder: embedding gather, residual add + RMSNorm (fused),
// SiLU(gate) * up.  The residual stream is float in both engines; norm sums, the
// activation and the residual sum are computed in 32-bit.
#include "common.h"

// h[m, :] = float(table[ids[m], :]).  An id outside [0, vocab) gives a row of NaN
// (the host refuses such a batch before anything runs).
__global__ void embed_gather_kernel(const int32_t* __restrict__ ids, const elem_t* __restrict__ table,
                                    float* __restrict__ h, int width, int vocab) {
    const int m = blockIdx.x;
    const int id = ids[m];
    float* out = h + (size_t)m * width;
    if (id < 0 || id >= vocab) {
        for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = __int_as_float(0x7fc00000);
        return;
    }
    const elem_t* row = table + (size_t)id * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = to_float(row[i]);
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < waves; ++i) total = fmaxf(total, scratch[i]);
    return total;
}

// A row whose sum of squares does not fit 32 bits (elements beyond about 1e19) or is no number: the
// reference's way of norming (src/minillm/cuda/ops.cu:87-126), the row divided by its largest element before
// it is squared, and eps scaled alike: largest = max(max |x|, sqrt(eps)), den = sqrt(mean((x / largest)^2) +
// eps / largest^2), y = ((x / largest) / den) * w; a row with an infinity or a NaN comes out as NaN.  The usual
// row never gets here, so it keeps its one pass and its bits.  x = hrow + drow (drow: what is still to be
// added, or null).  WAVE: one wavefront serves the row, else the whole workgroup (every thread of it must
// call, `scratch` holds 16 floats of LDS).
template <bool WAVE>
__device__ void norm_row_rescaled(const float* hrow, const elem_t* drow, const float* __restrict__ weight,
                                  elem_t* __restrict__ orow, int width, float eps, float* scratch) {
    __threadfence_block();                     // (the row may have been written back by other lanes just now)
    const int t = WAVE ? (int)(threadIdx.x & 63) : (int)threadIdx.x, step = WAVE ? 64 : (int)blockDim.x;
    float largest = 0.f;
    for (int i = t; i < width; i += step) {
        const float x = hrow[i] + (drow ? to_float(drow[i]) : 0.f);
        largest = fmaxf(largest, isfinite(x) ? fabsf(x) : INFINITY);
    }
    largest = WAVE ? wave_max(largest) : block_max(largest, scratch);
    largest = fmaxf(largest, sqrtf(eps));
    if (!isfinite(largest)) {
        for (int i = t; i < width; i += step) orow[i] = from_float<elem_t>(__int_as_float(0x7fc00000));
        return;
    }
    float sum = 0.f;
    for (int i = t; i < width; i += step) {
        const float scaled = (hrow[i] + (drow ? to_float(drow[i]) : 0.f)) / largest;
        sum += scaled * scaled;
    }
    sum = WAVE ? wave_sum(sum) : block_sum(sum, scratch);
    const float den = sqrtf(sum / (float)width + (eps / largest) / largest);
    for (int i = t; i < width; i += step) {
        const float x = hrow[i] + (drow ? to_float(drow[i]) : 0.f);
        orow[i] = from_float<elem_t>(((x / largest) / den) * weight[i]);
    }
}

// For output row r: src = rows ? rows[r] : r;  x = h[src] + (delta ? delta[src] : 0);
// if write_h: h[src] = x;  out[r] = (x * rsqrt(mean(x^2) + eps)) * weight.
// One workgroup per row; the sum of squares is taken over the row in a fixed order.
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                   const float* __restrict__ weight, elem_t* __restrict__ out,
                                   const int32_t* __restrict__ rows, int width, float eps,
                                   int write_h) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hrow = h + src * width;
    const elem_t* drow = delta ? delta + src * width : nullptr;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow) {
            x += to_float(drow[i]);
            if (write_h) hrow[i] = x;
        }
        sum += x * x;
    }
    sum = block_sum(sum, scratch);
    elem_t* orow = out + (size_t)r * width;
    if (!isfinite(sum)) {                      // (the same in every thread of the workgroup)
        norm_row_rescaled<false>(hrow, (drow && !write_h) ? drow : nullptr, weight, orow, width, eps, scratch);
        return;
    }
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow && !write_h) x += to_float(drow[i]);
        orow[i] = from_float<elem_t>((x * scale) * weight[i]);
    }
}

// One workgroup per row as above, 16 bytes per thread and access (width a multiple of MLR_VEC): for few
// rows of the bfloat16 engine, where the scalar kernel's latency would show.
__global__ __launch_bounds__(256) void add_rmsnorm_row_vec_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                                                  const float* __restrict__ weight,
                                                                  elem_t* __restrict__ out, const int32_t* __restrict__ rows,
                                                                  int width, float eps, int write_h) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hrow = h + src * width;
    const elem_t* drow = delta ? delta + src * width : nullptr;
    float sum = 0.f;
    for (int c = threadIdx.x * MLR_VEC; c < width; c += 256 * MLR_VEC) {
        float x[MLR_VEC];
#pragma unroll
        for (int e = 0; e < MLR_VEC; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(hrow + c + e);
            x[e] = v.x; x[e + 1] = v.y; x[e + 2] = v.z; x[e + 3] = v.w;
        }
        if (drow) {
            float dv[MLR_VEC];
            load_vec(drow + c, dv);
#pragma unroll
            for (int e = 0; e < MLR_VEC; ++e) x[e] += dv[e];
            if (write_h) {
#pragma unroll
                for (int e = 0; e < MLR_VEC; e += 4)
                    *reinterpret_cast<float4*>(hrow + c + e) = make_float4(x[e], x[e + 1], x[e + 2], x[e + 3]);
            }
        }
#pragma unroll
        for (int e = 0; e < MLR_VEC; ++e) sum += x[e] * x[e];
    }
    sum = block_sum(sum, scratch);
    elem_t* orow = out + (size_t)r * width;
    if (!isfinite(sum)) {
        norm_row_rescaled<false>(hrow, (drow && !write_h) ? drow : nullptr, weight, orow, width, eps, scratch);
        return;
    }
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    for (int c = threadIdx.x * MLR_VEC; c < width; c += 256 * MLR_VEC) {
        float x[MLR_VEC], y[MLR_VEC];
#pragma unroll
        for (int e = 0; e < MLR_VEC; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(hrow + c + e);
            x[e] = v.x; x[e + 1] = v.y; x[e + 2] = v.z; x[e + 3] = v.w;
        }
        if (drow && !write_h) {
            float dv[MLR_VEC];
            load_vec(drow + c, dv);
#pragma unroll
            for (int e = 0; e < MLR_VEC; ++e) x[e] += dv[e];
        }
#pragma unroll
        for (int e = 0; e < MLR_VEC; e += 4) {
            const float4 w = *reinterpret_cast<const float4*>(weight + c + e);
            y[e] = (x[e] * scale) * w.x;
            y[e + 1] = (x[e + 1] * scale) * w.y;
            y[e + 2] = (x[e + 2] * scale) * w.z;
            y[e + 3] = (x[e + 3] * scale) * w.w;
        }
        store_vec(orow + c, y);
    }
}

// The same for widths that are a multiple of 8 (bfloat16) or 4 (float), 16 bytes per lane and access:
// one wavefront per row, four rows per workgroup, the row kept in registers between the two passes
// when it fits (width <= 64 * MLR_VEC * ROW_REGS), else re-read.
#define ROW_REGS 4
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                                              const float* __restrict__ weight,
                                                              elem_t* __restrict__ out, const int32_t* __restrict__ rows,
                                                              int n_out, int width, float eps, int write_h) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= n_out) return;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hrow = h + src * width;
    const elem_t* drow = delta ? delta + src * width : nullptr;
    float x[ROW_REGS][MLR_VEC];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < ROW_REGS; ++i) {
        const int c = (lane + 64 * i) * MLR_VEC;
        if (c < width) {
#pragma unroll
            for (int e = 0; e < MLR_VEC; e += 4) {
                const float4 v = *reinterpret_cast<const float4*>(hrow + c + e);
                x[i][e] = v.x; x[i][e + 1] = v.y; x[i][e + 2] = v.z; x[i][e + 3] = v.w;
            }
            if (drow) {
                float dv[MLR_VEC];
                load_vec(drow + c, dv);
#pragma unroll
                for (int e = 0; e < MLR_VEC; ++e) x[i][e] += dv[e];
                if (write_h) {
#pragma unroll
                    for (int e = 0; e < MLR_VEC; e += 4)
                        *reinterpret_cast<float4*>(hrow + c + e) = make_float4(x[i][e], x[i][e + 1], x[i][e + 2], x[i][e + 3]);
                }
            }
#pragma unroll
            for (int e = 0; e < MLR_VEC; ++e) sum += x[i][e] * x[i][e];
        }
    }
    sum = wave_sum(sum);
    elem_t* orow = out + (size_t)r * width;
    if (!isfinite(sum)) {                      // (the same in every lane of the wavefront, which serves this row alone)
        norm_row_rescaled<true>(hrow, (drow && !write_h) ? drow : nullptr, weight, orow, width, eps, nullptr);
        return;
    }
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
#pragma unroll
    for (int i = 0; i < ROW_REGS; ++i) {
        const int c = (lane + 64 * i) * MLR_VEC;
        if (c < width) {
            float y[MLR_VEC];
#pragma unroll
            for (int e = 0; e < MLR_VEC; e += 4) {
                const float4 w = *reinterpret_cast<const float4*>(weight + c + e);
                y[e] = (x[i][e] * scale) * w.x;
                y[e + 1] = (x[i][e + 1] * scale) * w.y;
                y[e + 2] = (x[i][e + 2] * scale) * w.z;
                y[e + 3] = (x[i][e + 3] * scale) * w.w;
            }
            store_vec(orow + c, y);
        }
    }
}

// h[m, :] += delta[m, :] (the last residual sum when nothing is normed afterwards).
__global__ void residual_add_kernel(float* __restrict__ h, const elem_t* __restrict__ delta, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (size_t)gridDim.x * blockDim.x) {
        h[i] += to_float(delta[i]);
    }
}

// The activation of a gated feed-forward's gate: ACT 0 silu(g) = g / (1 + exp(-g)); ACT 1 the tanh form of gelu,
// 0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))).  32-bit.
template <int ACT>
__device__ __forceinline__ float gate_act(float g) {
    if (ACT == 1) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    return g / (1.0f + expf(-g));
}

// The same, 16 bytes per lane and access, for inter % MLR_VEC == 0.
template <int ACT>
__global__ void silu_mul_vec_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ act, int rows, int inter) {
    const int per_row = inter / MLR_VEC;
    const size_t total = (size_t)rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / per_row, f = (i % per_row) * MLR_VEC;
        float g[MLR_VEC], u[MLR_VEC], y[MLR_VEC];
        load_vec(gate_up + m * 2 * inter + f, g);
        load_vec(gate_up + m * 2 * inter + inter + f, u);
#pragma unroll
        for (int e = 0; e < MLR_VEC; ++e) y[e] = gate_act<ACT>(g[e]) * u[e];
        store_vec(act + m * inter + f, y);
    }
}

// act[m, f] = act(gate_up[m, f]) * gate_up[m, inter + f].
template <int ACT>
__global__ void silu_mul_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ act,
                                int rows, int inter) {
    const size_t total = (size_t)rows * inter;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / inter, f = i % inter;
        const float g = to_float(gate_up[m * 2 * inter + f]);
        const float u = to_float(gate_up[m * 2 * inter + inter + f]);
        act[i] = from_float<elem_t>(gate_act<ACT>(g) * u);
    }
}

// The embedding of a token plus the row of a pair table that the token and the one before it pick:
// h[m] = float(table[id]) + float(pairs[row]), row = (previous * mul_prev + id * mul_cur) mod buckets, and the table's
// last row (number `buckets`) for a request's first token (position 0).  The token before row m is the row above it
// when that row is the same request's previous position, else what the request's state holds (`live[slot]`); the
// last row that a request brings to the step leaves its token in `stage[slot]`.  An id outside [0, vocab) gives a
// row of NaN (the host refuses such a batch before anything runs).
__global__ void pair_embed_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ positions,
                                  const int32_t* __restrict__ slots, const elem_t* __restrict__ table,
                                  const elem_t* __restrict__ pairs, const int32_t* __restrict__ live,
                                  int32_t* __restrict__ stage, float* __restrict__ h, int rows, int width, int vocab,
                                  int buckets, long long mul_prev, long long mul_cur) {
    const int m = blockIdx.x;
    const int id = ids[m], pos = positions[m], slot = slots[m];
    float* out = h + (size_t)m * width;
    const bool last = m + 1 >= rows || slots[m + 1] != slot || positions[m + 1] != pos + 1;
    if (last && threadIdx.x == 0) stage[slot] = id;
    if (id < 0 || id >= vocab) {
        for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = __int_as_float(0x7fc00000);
        return;
    }
    long long pair = buckets;
    if (pos > 0) {
        const int before = m > 0 && slots[m - 1] == slot && positions[m - 1] == pos - 1 ? ids[m - 1] : live[slot];
        pair = ((long long)before * mul_prev + (long long)id * mul_cur) % buckets;
        if (pair < 0) pair += buckets;
    }
    const elem_t* row = table + (size_t)id * width;
    const elem_t* add = pairs + (size_t)pair * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = to_float(row[i]) + to_float(add[i]);
}

// out[m, c] = scale * x[m, c] * act(gate[m * gate_stride + c]); ACT 0 silu, 1 sigmoid.  32-bit inside.
template <int ACT>
__global__ void gate_mul_kernel(const elem_t* __restrict__ x, const elem_t* __restrict__ gate, long gate_stride,
                                elem_t* __restrict__ out, size_t rows, int width, float scale) {
    const size_t total = rows * width;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / width, c = i % width;
        const float g = to_float(gate[m * gate_stride + c]);
        const float s = 1.0f / (1.0f + expf(-g));
        out[i] = from_float<elem_t>(scale * (to_float(x[i]) * (ACT == 0 ? g * s : s)));
    }
}

// out[m] = x[m] / sqrt(mean(x[m]^2) + eps) * weight for a block of columns x[m * x_stride + c] of a wider matrix
// (a latent vector that comes out of a projection beside other things); 32-bit inside.  One workgroup a row.
__global__ __launch_bounds__(256) void rmsnorm_columns_kernel(const elem_t* __restrict__ x, long x_stride,
                                                              const float* __restrict__ weight, elem_t* __restrict__ out,
                                                              int width, float eps) {
    __shared__ float scratch[16];
    const elem_t* row = x + (size_t)blockIdx.x * x_stride;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float v = to_float(row[i]);
        sum += v * v;
    }
    const float r = 1.0f / sqrtf(block_sum(sum, scratch) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x)
        out[(size_t)blockIdx.x * width + i] = from_float<elem_t>((to_float(row[i]) * r) * weight[i]);
}

// out = sa * a + sb * b, the sum taken in 32-bit.
__global__ void scaled_sum_kernel(const elem_t* __restrict__ a, const elem_t* __restrict__ b, elem_t* __restrict__ out,
                                  float sa, float sb, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        out[i] = from_float<elem_t>(sa * to_float(a[i]) + sb * to_float(b[i]));
}

// The first half of an RMSNorm whose scale is applied by the projection that follows (few rows): x = h + delta
// (delta may be null; written back to h when write_h), out = elem(x * weight) WITHOUT the scale, and the row's
// sum of squares ss[r] (one "partial" sum a row).  One workgroup per row, sums in a fixed order.
__global__ void rows_prenorm_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                    const float* __restrict__ weight, elem_t* __restrict__ out,
                                    float* __restrict__ ss, int width) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    float* hrow = h + (size_t)r * width;
    const elem_t* drow = delta ? delta + (size_t)r * width : nullptr;
    elem_t* orow = out + (size_t)r * width;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow) {
            x += to_float(drow[i]);
            hrow[i] = x;
        }
        sum += x * x;
        orow[i] = from_float<elem_t>(x * weight[i]);
    }
    sum = block_sum(sum, scratch);
    if (threadIdx.x == 0) ss[r] = sum;
}

// The check of the hidden state (a debug mode; the reference runs the like after every layer and poisons
// its runtime, src/minillm/cuda/layer.cpp:71, src/minillm/cuda/ops.cu:29-43).  status[0] collects bits
// (1: a NaN, 2: an infinity), status[1] the smallest (layer << 20 | row) at which one was seen.
__global__ void status_reset_kernel(int32_t* __restrict__ status) {
    if (threadIdx.x == 0) {
        status[0] = 0;
        status[1] = 0x7fffffff;
    }
}

// One workgroup per row of x = h + delta (delta may be null): which kinds of non-finite values it holds.
__global__ void finite_check_kernel(const float* __restrict__ h, const elem_t* __restrict__ delta, int width, int layer,
                                    int32_t* __restrict__ status) {
    const int r = blockIdx.x;
    const float* hrow = h + (size_t)r * width;
    const elem_t* drow = delta ? delta + (size_t)r * width : nullptr;
    int bits = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float x = hrow[i] + (drow ? to_float(drow[i]) : 0.f);
        const uint32_t u = __float_as_uint(x) & 0x7fffffffu;
        if (u > 0x7f800000u) bits |= 1;
        else if (u == 0x7f800000u) bits |= 2;
    }
    if (__any(bits != 0)) {                     // (rare: one atomic per wavefront that saw something)
        for (int off = 32; off > 0; off >>= 1) bits |= __shfl_xor(bits, off, MLR_WAVE);
        if ((threadIdx.x & 63) == 0) {
            atomicOr(&status[0], bits);
            atomicMin(&status[1], (layer << 20) | (r < (1 << 20) ? r : (1 << 20) - 1));
        }
    }
}


// A layer whose mixer and feed-forward read the SAME input through norms of their own: x = h + d1 + d2 (what
// the layer before still has to add; either may be null), written back to h; out1 = (x * r) * w1 and
// out2 = (x * r) * w2 with the one r = rsqrt(mean(x^2) + eps) that both norms share (out2 / w2 may be null).
// One workgroup per row, the sum of squares in a fixed order.
__global__ void add2_rmsnorm2_kernel(float* __restrict__ h, const elem_t* __restrict__ d1, const elem_t* __restrict__ d2,
                                     const float* __restrict__ w1, const float* __restrict__ w2,
                                     elem_t* __restrict__ out1, elem_t* __restrict__ out2, int width, float eps) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float* hrow = h + r * width;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (d1 || d2) {
            float add = d1 ? to_float(d1[r * width + i]) : 0.f;
            if (d2) add += to_float(d2[r * width + i]);
            x += add;
            hrow[i] = x;
        }
        sum += x * x;
    }
    sum = block_sum(sum, scratch);
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float x = hrow[i] * scale;           // (this thread wrote hrow[i] itself)
        out1[r * width + i] = from_float<elem_t>(x * w1[i]);
        if (out2) out2[r * width + i] = from_float<elem_t>(x * w2[i]);
    }
}

// h += d1 + d2 (d2 may be null): the two branches of such a layer added in 32-bit when no norm follows.
__global__ void residual_add2_kernel(float* __restrict__ h, const elem_t* __restrict__ d1, const elem_t* __restrict__ d2,
                                     size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
        float add = to_float(d1[i]);
        if (d2) add += to_float(d2[i]);
        h[i] += add;
    }
}

// act[m, f] = g * sigmoid(slope * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit);
// gate = gate_up[m, f], up = gate_up[m, inter + f].
__global__ void clamped_glu_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ act, int rows, int inter,
                                   float limit, float slope) {
    const size_t total = (size_t)rows * inter;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / inter, f = i % inter;
        const float g = fminf(to_float(gate_up[m * 2 * inter + f]), limit);
        const float u = fminf(fmaxf(to_float(gate_up[m * 2 * inter + inter + f]), -limit), limit);
        act[i] = from_float<elem_t>((g / (1.0f + expf(-slope * g))) * (u + 1.0f));
    }
}

// The end of a recurrent mixer: y [rows, width] float is cut into parts of `part` values, each divided by its
// own root mean square (eps inside the root) and multiplied by weight[i % period]; the gate (an activation of
// gate[m, i], read with a row stride of its own) multiplies before the norm (gate_first) or after it.
// One wavefront per (row, part); gate_kind 0: silu, 1: sigmoid.
__global__ __launch_bounds__(256) void gated_part_norm_kernel(const float* __restrict__ y, const elem_t* __restrict__ gate,
                                                              long gate_stride, const float* __restrict__ weight,
                                                              elem_t* __restrict__ out, int rows, int width, int part,
                                                              int period, float eps, int gate_first, int gate_kind) {
    const int lane = threadIdx.x & 63;
    const size_t unit = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const int parts = width / part;
    if (unit >= (size_t)rows * parts) return;
    const size_t m = unit / parts;
    const int c0 = (int)(unit % parts) * part;
    const float* yrow = y + m * width;
    const elem_t* grow = gate + m * gate_stride;
    auto gate_of = [&](int c) {
        const float z = to_float(grow[c]);
        const float s = 1.0f / (1.0f + expf(-z));
        return gate_kind == 0 ? z * s : s;
    };
    float sum = 0.f;
    for (int i = lane; i < part; i += 64) {
        float v = yrow[c0 + i];
        if (gate_first) v *= gate_of(c0 + i);
        sum += v * v;
    }
    sum = wave_sum(sum);
    const float scale = 1.0f / sqrtf(sum / (float)part + eps);
    for (int i = lane; i < part; i += 64) {
        const int c = c0 + i;
        float v = yrow[c];
        if (gate_first) v *= gate_of(c);
        v = (v * scale) * weight[c % period];
        if (!gate_first) v *= gate_of(c);
        out[m * width + c] = from_float<elem_t>(v);
    }
}

#if MLR_BF16
// The same three kernels with 16 bytes per lane and access (bfloat16 engine, widths in multiples of 8).
__global__ __launch_bounds__(256) void add2_rmsnorm2_vec_kernel(float* __restrict__ h, const elem_t* __restrict__ d1,
                                                                const elem_t* __restrict__ d2, const float* __restrict__ w1,
                                                                const float* __restrict__ w2, elem_t* __restrict__ out1,
                                                                elem_t* __restrict__ out2, int width, float eps) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float* hrow = h + r * width;
    float sum = 0.f;
    for (int c = threadIdx.x * 8; c < width; c += 256 * 8) {
        float x[8], a[8];
        const float4 lo = *reinterpret_cast<const float4*>(hrow + c), hi = *reinterpret_cast<const float4*>(hrow + c + 4);
        x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w; x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
        if (d1 || d2) {
            if (d1) load_vec(d1 + r * width + c, a);
            else {
#pragma unroll
                for (int e = 0; e < 8; ++e) a[e] = 0.f;
            }
            if (d2) {
                float b[8];
                load_vec(d2 + r * width + c, b);
#pragma unroll
                for (int e = 0; e < 8; ++e) a[e] += b[e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) x[e] += a[e];
            *reinterpret_cast<float4*>(hrow + c) = make_float4(x[0], x[1], x[2], x[3]);
            *reinterpret_cast<float4*>(hrow + c + 4) = make_float4(x[4], x[5], x[6], x[7]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += x[e] * x[e];
    }
    sum = block_sum(sum, scratch);
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    for (int c = threadIdx.x * 8; c < width; c += 256 * 8) {       // (this thread wrote these elements of h itself)
        float x[8], y[8];
        const float4 lo = *reinterpret_cast<const float4*>(hrow + c), hi = *reinterpret_cast<const float4*>(hrow + c + 4);
        x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w; x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = (x[e] * scale) * w1[c + e];
        store_vec(out1 + r * width + c, y);
        if (out2) {
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = (x[e] * scale) * w2[c + e];
            store_vec(out2 + r * width + c, y);
        }
    }
}

__global__ void clamped_glu_vec_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ act, int rows, int inter,
                                       float limit, float slope) {
    const int per_row = inter / 8;
    const size_t total = (size_t)rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / per_row, f = (i % per_row) * 8;
        float g[8], u[8], y[8];
        load_vec(gate_up + m * 2 * inter + f, g);
        load_vec(gate_up + m * 2 * inter + inter + f, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float gg = fminf(g[e], limit), uu = fminf(fmaxf(u[e], -limit), limit);
            y[e] = (gg / (1.0f + expf(-slope * gg))) * (uu + 1.0f);
        }
        store_vec(act + m * inter + f, y);
    }
}

// WAVES wavefronts per (row, part): one for short parts, four (a workgroup) for long ones.
template <int WAVES>
__global__ __launch_bounds__(256) void gated_part_norm_vec_kernel(const float* __restrict__ y, const elem_t* __restrict__ gate,
                                                                  long gate_stride, const float* __restrict__ weight,
                                                                  elem_t* __restrict__ out, int rows, int width, int part,
                                                                  int period, float eps, int gate_first, int gate_kind) {
    __shared__ float scratch[16];
    const int lane = WAVES == 1 ? (int)(threadIdx.x & 63) : (int)threadIdx.x;
    const size_t unit = WAVES == 1 ? (size_t)blockIdx.x * 4 + (threadIdx.x >> 6) : (size_t)blockIdx.x;
    const int parts = width / part;
    const bool live = unit < (size_t)rows * parts;
    const size_t m = live ? unit / parts : 0;
    const int c0 = live ? (int)(unit % parts) * part : 0;
    const float* yrow = y + m * width;
    const elem_t* grow = gate + m * gate_stride;
    auto gated = [&](int c, float* v, bool before) {        // v = y[c .. c + 8), times the gate's activation when `before`
        const float4 lo = *reinterpret_cast<const float4*>(yrow + c), hi = *reinterpret_cast<const float4*>(yrow + c + 4);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
        float z[8];
        load_vec(grow + c, z);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float sg = 1.0f / (1.0f + expf(-z[e]));
            z[e] = gate_kind == 0 ? z[e] * sg : sg;
            if (before) v[e] *= z[e];
        }
        if (!before) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = z[e];         // (the caller wants the gate itself)
        }
    };
    float sum = 0.f;
    if (live)
        for (int i = lane * 8; i < part; i += 64 * WAVES * 8) {
            float v[8];
            if (gate_first) gated(c0 + i, v, true);
            else {
                const float4 lo = *reinterpret_cast<const float4*>(yrow + c0 + i), hi = *reinterpret_cast<const float4*>(yrow + c0 + i + 4);
                v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) sum += v[e] * v[e];
        }
    sum = WAVES == 1 ? wave_sum(sum) : block_sum(sum, scratch);
    if (!live) return;
    const float scale = 1.0f / sqrtf(sum / (float)part + eps);
    for (int i = lane * 8; i < part; i += 64 * WAVES * 8) {
        const int c = c0 + i;
        float v[8], o[8];
        if (gate_first) {
            gated(c, v, true);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (v[e] * scale) * weight[(c + e) % period];
        } else {
            float gt[8];
            gated(c, gt, false);
            const float4 lo = *reinterpret_cast<const float4*>(yrow + c), hi = *reinterpret_cast<const float4*>(yrow + c + 4);
            v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = ((v[e] * scale) * weight[(c + e) % period]) * gt[e];
        }
        store_vec(out + m * width + c, o);
    }
}
#endif

// Layer norm of a row, y = (x - mean) / sqrt(var + eps) * weight + bias with var the mean of the squared
// deviations (two passes over the row, 32-bit), times `out_scale`.  The row comes from `xe` (the engine's element
// type) or from `xf` (float), whichever is not null; for output row r it is row src = rows ? rows[r] : r.
//   acc != null: acc[src] += y (the float residual stream takes a sublayer's normed output), and with
//     cast != null also cast[src] = T(acc[src]): the stream as the next sublayer's input;
//   else out[r] = T(y).
// One workgroup a row.
#define LN_REGS 16
__global__ __launch_bounds__(256) void layernorm_kernel(const elem_t* __restrict__ xe, const float* __restrict__ xf,
                                                        const float* __restrict__ weight, const float* __restrict__ bias,
                                                        const int32_t* __restrict__ rows, float* __restrict__ acc,
                                                        elem_t* __restrict__ cast, elem_t* __restrict__ out, int width,
                                                        float eps, float out_scale) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    const elem_t* re = xe ? xe + src * width : nullptr;
    const float* rf = xf ? xf + src * width : nullptr;
    // the row is read once and kept in registers where it fits (up to LN_REGS values a thread), else read again
    const bool kept = width <= LN_REGS * (int)blockDim.x;
    float x[LN_REGS];
    float sum = 0.f;
    if (kept) {
#pragma unroll
        for (int j = 0; j < LN_REGS; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            x[j] = i < width ? (re ? to_float(re[i]) : rf[i]) : 0.f;
            sum += x[j];
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) sum += re ? to_float(re[i]) : rf[i];
    }
    const float mean = block_sum(sum, scratch) / (float)width;
    float dev = 0.f;
    if (kept) {
#pragma unroll
        for (int j = 0; j < LN_REGS; ++j) {
            const float d = threadIdx.x + j * blockDim.x < width ? x[j] - mean : 0.f;
            dev += d * d;
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) {
            const float d = (re ? to_float(re[i]) : rf[i]) - mean;
            dev += d * d;
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(dev, scratch) / (float)width + eps);
    auto finish = [&](int i, float xv) {
        const float y = (((xv - mean) * inv) * weight[i] + (bias ? bias[i] : 0.f)) * out_scale;
        if (acc != nullptr) {
            const float sumh = acc[src * width + i] + y;
            acc[src * width + i] = sumh;
            if (cast != nullptr) cast[src * width + i] = from_float<elem_t>(sumh);
        } else {
            out[(size_t)r * width + i] = from_float<elem_t>(y);
        }
    };
    if (kept) {
#pragma unroll
        for (int j = 0; j < LN_REGS; ++j) {
            const int i = threadIdx.x + j * blockDim.x;
            if (i < width) finish(i, x[j]);
        }
    } else {
        for (int i = threadIdx.x; i < width; i += blockDim.x) finish(i, re ? to_float(re[i]) : rf[i]);
    }
}

// out = relu(x)^2, element by element (32-bit).
__global__ void relu_squared_kernel(const elem_t* __restrict__ x, elem_t* __restrict__ out, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) {
        const float r = fmaxf(to_float(x[i]), 0.f);
        out[i] = from_float<elem_t>(r * r);
    }
}

// out = T(h): the float residual stream as a sublayer's input.
__global__ void cast_rows_kernel(const float* __restrict__ h, elem_t* __restrict__ out, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        out[i] = from_float<elem_t>(h[i]);
}

// x *= factor (float values, logits for instance).
__global__ void scale_float_kernel(float* __restrict__ x, float factor, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        x[i] *= factor;
}

// ---- a norm without statistics: y = tanh(alpha x) w + b, element by element, 32-bit ---------------------------
__device__ __forceinline__ float tanh_norm(float x, float alpha, float w, float b) { return __builtin_fmaf(tanhf(alpha * x), w, b); }

// VEC consecutive values in one access where VEC is 4 (the row's width a multiple of 4: 16-byte float accesses, 8- or
// 16-byte accesses of the engine's element type), else one by one.
template <int VEC> __device__ __forceinline__ void load_floats(const float* p, float* out) {
    if (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    } else {
        out[0] = p[0];
    }
}
template <int VEC> __device__ __forceinline__ void store_floats(float* p, const float* in) {
    if (VEC == 4) *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
    else p[0] = in[0];
}
template <int VEC> __device__ __forceinline__ void load_elems(const elem_t* p, float* out) {
    if (VEC == 4) {
#if MLR_BF16
        const uint2 v = *reinterpret_cast<const uint2*>(p);
        out[0] = __uint_as_float(v.x << 16); out[1] = __uint_as_float(v.x & 0xffff0000u);
        out[2] = __uint_as_float(v.y << 16); out[3] = __uint_as_float(v.y & 0xffff0000u);
#else
        load_floats<4>(p, out);
#endif
    } else {
        out[0] = to_float(p[0]);
    }
}
template <int VEC> __device__ __forceinline__ void store_elems(elem_t* p, const float* in) {
    if (VEC == 4) {
#if MLR_BF16
        alignas(8) elem_t tmp[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) tmp[e] = from_float<elem_t>(in[e]);
        *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(tmp);
#else
        store_floats<4>(p, in);
#endif
    } else {
        p[0] = from_float<elem_t>(in[0]);
    }
}

// x = h[row] + delta[row] (delta may be null; written back to h when write_h), out[r] = norm(x) for row = rows[r]
// (rows null: r).  One thread takes VEC consecutive elements (width a multiple of VEC).
template <int VEC>
__global__ void tanh_norm_rows_kernel(float* __restrict__ h, const elem_t* __restrict__ delta, const float* __restrict__ w,
                                      const float* __restrict__ b, float alpha, elem_t* __restrict__ out,
                                      const int32_t* __restrict__ rows, size_t n_out, int width, int write_h) {
    const size_t per_row = width / VEC, total = n_out * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t r = i / per_row, c = (i % per_row) * VEC;
        const size_t row = rows != nullptr ? (size_t)rows[r] : r;
        float x[VEC], d[VEC], wv[VEC], bv[VEC], y[VEC];
        load_floats<VEC>(h + row * width + c, x);
        if (delta != nullptr) {
            load_elems<VEC>(delta + row * width + c, d);
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[e] += d[e];
            if (write_h) store_floats<VEC>(h + row * width + c, x);
        }
        load_floats<VEC>(w + c, wv);
        load_floats<VEC>(b + c, bv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) y[e] = tanh_norm(x[e], alpha, wv[e], bv[e]);
        store_elems<VEC>(out + r * width + c, y);
    }
}

// h += norm_a(delta) (+ extra, a float matrix like h, when given); then, when out is given, out = norm_n(h): the norm
// behind a sublayer, the residual sum and the norm in front of the next sublayer in one pass over the row.
template <int VEC>
__global__ void tanh_norm_add_kernel(const elem_t* __restrict__ delta, const float* __restrict__ wa, const float* __restrict__ ba,
                                     float alpha_a, float* __restrict__ h, const float* __restrict__ extra,
                                     const float* __restrict__ wn, const float* __restrict__ bn, float alpha_n,
                                     elem_t* __restrict__ out, size_t n_rows, int width) {
    const size_t per_row = width / VEC, total = n_rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t at = (i / per_row) * width + (i % per_row) * VEC;
        const int c = (int)((i % per_row) * VEC);
        float x[VEC], d[VEC], wv[VEC], bv[VEC], ev[VEC], y[VEC];
        load_floats<VEC>(h + at, x);
        load_elems<VEC>(delta + at, d);
        load_floats<VEC>(wa + c, wv);
        load_floats<VEC>(ba + c, bv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] += tanh_norm(d[e], alpha_a, wv[e], bv[e]);
        if (extra != nullptr) {
            load_floats<VEC>(extra + at, ev);
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[e] += ev[e];
        }
        store_floats<VEC>(h + at, x);
        if (out != nullptr) {
            load_floats<VEC>(wn + c, wv);
            load_floats<VEC>(bn + c, bv);
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[e] = tanh_norm(x[e], alpha_n, wv[e], bv[e]);
            store_elems<VEC>(out + at, y);
        }
    }
}

// h += extra (float matrices of the same size).
__global__ void residual_add_float_kernel(float* __restrict__ h, const float* __restrict__ extra, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        h[i] += extra[i];
}

// dst = src (float matrices of the same size): the copy of the residual stream that later passes add again.
__global__ void copy_float_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

// x <- cap * tanh(x / cap) (float values, logits for instance).
__global__ void tanh_cap_kernel(float* __restrict__ x, float cap, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        x[i] = cap * tanhf(x[i] / cap);
}

// out[m, head * part + c] = x[m, head * part + c] * sigmoid(gate[m * gate_stride + head]): one gate a head.
__global__ void head_gate_mul_kernel(const elem_t* __restrict__ x, const elem_t* __restrict__ gate, long gate_stride,
                                     elem_t* __restrict__ out, size_t rows, int width, int part) {
    const size_t total = rows * width;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / width, c = i % width;
        const float g = to_float(gate[m * gate_stride + c / part]);
        out[i] = from_float<elem_t>(to_float(x[i]) / (1.0f + expf(-g)));
    }
}

static int grid_for(size_t count, int block) {
    size_t g = (count + block - 1) / block;
    return (int)(g > 65535 ? 65535 : (g == 0 ? 1 : g));
}

template <int ACT>
static int launch_gated(const void* gate_up, void* act, int rows, int inter, hipStream_t stream) {
    if (inter % MLR_VEC == 0) {
        silu_mul_vec_kernel<ACT><<<grid_for((size_t)rows * (inter / MLR_VEC), 256), 256, 0, stream>>>(
            (const elem_t*)gate_up, (elem_t*)act, rows, inter);
        return (int)hipGetLastError();
    }
    silu_mul_kernel<ACT><<<grid_for((size_t)rows * inter, 256), 256, 0, stream>>>(
        (const elem_t*)gate_up, (elem_t*)act, rows, inter);
    return (int)hipGetLastError();
}

// Whether every pointer given (null ones aside) allows 16-byte accesses.
template <class... P> static bool aligned16(P... pointers) {
    return (((uintptr_t)pointers % 16 == 0) && ...);
}

extern "C" {

int mlr_embed_gather(const int32_t* ids, const void* table, float* h, int rows, int width, int vocab,
                     hipStream_t stream) {
    if (rows <= 0) return 0;
    embed_gather_kernel<<<rows, 256, 0, stream>>>(ids, (const elem_t*)table, h, width, vocab);
    return (int)hipGetLastError();
}

int mlr_add_rmsnorm(float* h, const void* delta, const float* weight, void* out, const int32_t* rows,
                    int n_out, int width, float eps, int write_h, hipStream_t stream) {
    if (n_out <= 0) return 0;
    // (the float engine keeps its one order of additions for every batch size)
    if (MLR_BF16 && width % MLR_VEC == 0 && width <= 64 * MLR_VEC * ROW_REGS && n_out >= 64) {
        add_rmsnorm_vec_kernel<<<(n_out + 3) / 4, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out,
                                                                     rows, n_out, width, eps, write_h);
        return (int)hipGetLastError();
    }
    if (MLR_BF16 && width % MLR_VEC == 0) {
        add_rmsnorm_row_vec_kernel<<<n_out, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, rows,
                                                              width, eps, write_h);
        return (int)hipGetLastError();
    }
    add_rmsnorm_kernel<<<n_out, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, rows,
                                                  width, eps, write_h);
    return (int)hipGetLastError();
}

int mlr_rows_prenorm(float* h, const void* delta, const float* weight, void* out, float* ss, int rows, int width,
                     hipStream_t stream) {
    if (rows <= 0) return 0;
    rows_prenorm_kernel<<<rows, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, ss, width);
    return (int)hipGetLastError();
}

int mlr_status_reset(int32_t* status, hipStream_t stream) {
    status_reset_kernel<<<1, 64, 0, stream>>>(status);
    return (int)hipGetLastError();
}

int mlr_finite_check(const float* h, const void* delta, int rows, int width, int layer, int32_t* status,
                     hipStream_t stream) {
    if (rows <= 0) return 0;
    if (layer < 0 || layer >= 2047) return -1;
    finite_check_kernel<<<rows, 256, 0, stream>>>(h, (const elem_t*)delta, width, layer, status);
    return (int)hipGetLastError();
}

int mlr_residual_add(float* h, const void* delta, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    residual_add_kernel<<<grid_for(count, 256), 256, 0, stream>>>(h, (const elem_t*)delta, count);
    return (int)hipGetLastError();
}

int mlr_silu_mul(const void* gate_up, void* act, int rows, int inter, hipStream_t stream) {
    if (rows <= 0) return 0;
    return launch_gated<0>(gate_up, act, rows, inter, stream);
}

// act = activation(gate) * up; kind 0: silu, 1: the tanh form of gelu
int mlr_gated_act_mul(const void* gate_up, void* act, int rows, int inter, int kind, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (kind == 0) return launch_gated<0>(gate_up, act, rows, inter, stream);
    if (kind == 1) return launch_gated<1>(gate_up, act, rows, inter, stream);
    return -1;
}

int mlr_pair_embed(const int32_t* ids, const int32_t* positions, const int32_t* slots, const void* table, const void* pairs,
                   const int32_t* live, int32_t* stage, float* h, int rows, int width, int vocab, int buckets,
                   long long mul_prev, long long mul_cur, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (buckets < 1) return -1;
    pair_embed_kernel<<<rows, 256, 0, stream>>>(ids, positions, slots, (const elem_t*)table, (const elem_t*)pairs, live, stage,
                                                h, rows, width, vocab, buckets, mul_prev, mul_cur);
    return (int)hipGetLastError();
}

// out = scale * x * act(gate); kind 0: silu, 1: sigmoid; gate: columns of a row-major matrix
int mlr_gate_mul(const void* x, const void* gate, long gate_stride, void* out, int rows, int width, int kind, float scale,
                 hipStream_t stream) {
    if (rows <= 0 || width <= 0) return 0;
    const int grid = grid_for((size_t)rows * width, 256);
    if (kind == 0)
        gate_mul_kernel<0><<<grid, 256, 0, stream>>>((const elem_t*)x, (const elem_t*)gate, gate_stride, (elem_t*)out,
                                                     (size_t)rows, width, scale);
    else if (kind == 1)
        gate_mul_kernel<1><<<grid, 256, 0, stream>>>((const elem_t*)x, (const elem_t*)gate, gate_stride, (elem_t*)out,
                                                     (size_t)rows, width, scale);
    else
        return -1;
    return (int)hipGetLastError();
}

int mlr_rmsnorm_columns(const void* x, long x_stride, const float* weight, void* out, int rows, int width, float eps,
                        hipStream_t stream) {
    if (rows <= 0 || width <= 0) return 0;
    rmsnorm_columns_kernel<<<rows, 256, 0, stream>>>((const elem_t*)x, x_stride, weight, (elem_t*)out, width, eps);
    return (int)hipGetLastError();
}

int mlr_scaled_sum(const void* a, const void* b, void* out, float sa, float sb, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    scaled_sum_kernel<<<grid_for(count, 256), 256, 0, stream>>>((const elem_t*)a, (const elem_t*)b, (elem_t*)out, sa, sb, count);
    return (int)hipGetLastError();
}

int mlr_add2_rmsnorm2(float* h, const void* d1, const void* d2, const float* w1, const float* w2, void* out1, void* out2,
                      int rows, int width, float eps, hipStream_t stream) {
    if (rows <= 0) return 0;
    if ((out2 == nullptr) != (w2 == nullptr)) return -1;
#if MLR_BF16
    if (width % 8 == 0) {
        add2_rmsnorm2_vec_kernel<<<rows, 256, 0, stream>>>(h, (const elem_t*)d1, (const elem_t*)d2, w1, w2, (elem_t*)out1,
                                                           (elem_t*)out2, width, eps);
        return (int)hipGetLastError();
    }
#endif
    add2_rmsnorm2_kernel<<<rows, 256, 0, stream>>>(h, (const elem_t*)d1, (const elem_t*)d2, w1, w2, (elem_t*)out1,
                                                   (elem_t*)out2, width, eps);
    return (int)hipGetLastError();
}

int mlr_residual_add2(float* h, const void* d1, const void* d2, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    residual_add2_kernel<<<grid_for(count, 256), 256, 0, stream>>>(h, (const elem_t*)d1, (const elem_t*)d2, count);
    return (int)hipGetLastError();
}

int mlr_clamped_glu(const void* gate_up, void* act, int rows, int inter, float limit, float slope, hipStream_t stream) {
    if (rows <= 0) return 0;
#if MLR_BF16
    if (inter % 8 == 0) {
        clamped_glu_vec_kernel<<<grid_for((size_t)rows * (inter / 8), 256), 256, 0, stream>>>((const elem_t*)gate_up, (elem_t*)act,
                                                                                            rows, inter, limit, slope);
        return (int)hipGetLastError();
    }
#endif
    clamped_glu_kernel<<<grid_for((size_t)rows * inter, 256), 256, 0, stream>>>((const elem_t*)gate_up, (elem_t*)act, rows,
                                                                              inter, limit, slope);
    return (int)hipGetLastError();
}

int mlr_gated_part_norm(const float* y, const void* gate, long gate_stride, const float* weight, void* out, int rows,
                        int width, int part, int period, float eps, int gate_first, int gate_kind, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (part <= 0 || width % part != 0 || period <= 0) return -1;
    const size_t units = (size_t)rows * (width / part);
#if MLR_BF16
    // (16-byte accesses: parts, the gate's rows and its first column at multiples of 8 elements)
    if (part % 8 == 0 && gate_stride % 8 == 0 && ((uintptr_t)gate) % 16 == 0 && units < (1u << 31)) {
        if (part >= 2048)
            gated_part_norm_vec_kernel<4><<<(unsigned)units, 256, 0, stream>>>(y, (const elem_t*)gate, gate_stride, weight,
                                                                              (elem_t*)out, rows, width, part, period, eps,
                                                                              gate_first, gate_kind);
        else
            gated_part_norm_vec_kernel<1><<<(unsigned)((units + 3) / 4), 256, 0, stream>>>(y, (const elem_t*)gate, gate_stride,
                                                                                          weight, (elem_t*)out, rows, width,
                                                                                          part, period, eps, gate_first,
                                                                                          gate_kind);
        return (int)hipGetLastError();
    }
#endif
    gated_part_norm_kernel<<<(unsigned)((units + 3) / 4), 256, 0, stream>>>(y, (const elem_t*)gate, gate_stride, weight,
                                                                           (elem_t*)out, rows, width, part, period, eps,
                                                                           gate_first, gate_kind);
    return (int)hipGetLastError();
}

int mlr_layernorm(const void* xe, const float* xf, const float* weight, const float* bias, const int32_t* rows, float* acc,
                  void* cast, void* out, int n_out, int width, float eps, float out_scale, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if ((xe == nullptr) == (xf == nullptr) || (acc == nullptr && out == nullptr) || (acc != nullptr && rows != nullptr))
        return -1;
    layernorm_kernel<<<n_out, 256, 0, stream>>>((const elem_t*)xe, xf, weight, bias, rows, acc, (elem_t*)cast,
                                                (elem_t*)out, width, eps, out_scale);
    return (int)hipGetLastError();
}

int mlr_relu_squared(const void* x, void* out, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    relu_squared_kernel<<<grid_for(count, 256), 256, 0, stream>>>((const elem_t*)x, (elem_t*)out, count);
    return (int)hipGetLastError();
}

int mlr_cast_rows(const float* h, void* out, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    cast_rows_kernel<<<grid_for(count, 256), 256, 0, stream>>>(h, (elem_t*)out, count);
    return (int)hipGetLastError();
}

// out[r] = tanh(alpha (h + delta)[rows[r] or r]) w + b; h += delta when write_h
int mlr_tanh_norm_rows(float* h, const void* delta, const float* w, const float* b, float alpha, void* out,
                       const int32_t* rows, int n_out, int width, int write_h, hipStream_t stream) {
    if (n_out <= 0 || width <= 0) return 0;
    if (width % 4 == 0 && aligned16(h, delta, w, b, out))
        tanh_norm_rows_kernel<4><<<grid_for((size_t)n_out * (width / 4), 256), 256, 0, stream>>>(
            h, (const elem_t*)delta, w, b, alpha, (elem_t*)out, rows, (size_t)n_out, width, write_h);
    else
        tanh_norm_rows_kernel<1><<<grid_for((size_t)n_out * width, 256), 256, 0, stream>>>(
            h, (const elem_t*)delta, w, b, alpha, (elem_t*)out, rows, (size_t)n_out, width, write_h);
    return (int)hipGetLastError();
}

// h += tanh(alpha_a delta) wa + ba (+ extra); out (may be null) = tanh(alpha_n h) wn + bn
int mlr_tanh_norm_add(const void* delta, const float* wa, const float* ba, float alpha_a, float* h, const float* extra,
                      const float* wn, const float* bn, float alpha_n, void* out, int rows, int width, hipStream_t stream) {
    if (rows <= 0 || width <= 0) return 0;
    if (out != nullptr && (wn == nullptr || bn == nullptr)) return -1;
    if (width % 4 == 0 && aligned16(delta, wa, ba, h, extra) && aligned16(wn, bn, out))
        tanh_norm_add_kernel<4><<<grid_for((size_t)rows * (width / 4), 256), 256, 0, stream>>>(
            (const elem_t*)delta, wa, ba, alpha_a, h, extra, wn, bn, alpha_n, (elem_t*)out, (size_t)rows, width);
    else
        tanh_norm_add_kernel<1><<<grid_for((size_t)rows * width, 256), 256, 0, stream>>>(
            (const elem_t*)delta, wa, ba, alpha_a, h, extra, wn, bn, alpha_n, (elem_t*)out, (size_t)rows, width);
    return (int)hipGetLastError();
}

int mlr_residual_add_float(float* h, const float* extra, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    residual_add_float_kernel<<<grid_for(count, 256), 256, 0, stream>>>(h, extra, count);
    return (int)hipGetLastError();
}

int mlr_copy_float(const float* src, float* dst, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    copy_float_kernel<<<grid_for(count, 256), 256, 0, stream>>>(src, dst, count);
    return (int)hipGetLastError();
}

int mlr_tanh_cap(float* x, float cap, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    if (!(cap > 0.f)) return -1;
    tanh_cap_kernel<<<grid_for(count, 256), 256, 0, stream>>>(x, cap, count);
    return (int)hipGetLastError();
}

int mlr_head_gate_mul(const void* x, const void* gate, long gate_stride, void* out, int rows, int width, int part,
                      hipStream_t stream) {
    if (rows <= 0 || width <= 0) return 0;
    if (part < 1 || width % part != 0) return -1;
    head_gate_mul_kernel<<<grid_for((size_t)rows * width, 256), 256, 0, stream>>>((const elem_t*)x, (const elem_t*)gate,
                                                                                 gate_stride, (elem_t*)out, (size_t)rows, width, part);
    return (int)hipGetLastError();
}

int mlr_scale_float(float* x, float factor, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    scale_float_kernel<<<grid_for(count, 256), 256, 0, stream>>>(x, factor, count);
    return (int)hipGetLastError();
}

}  // extern "C"
