// Kernels around a residual stream that is kept in 32-bit whatever the compute type is:
// layer norm (weight, no bias) with the pending branch outputs added first and one or two
// normalised copies written, the join of the stream with a second tensor in front of a product,
// the gated activation with a choice of activation, and a per-head sigmoid gate.
//
// Storage types are run-time codes (KVA_F32 / KVA_BF16) per operand: the stream may be fp32 while
// the branch outputs and the normalised rows are bf16.  All arithmetic is fp32; sums over a row
// are taken in a fixed order, so a row's result does not depend on the other rows of the launch.
#include "common.h"
#include <math.h>

__device__ inline float ld_as_float(const void *p, int dtype, size_t i) {
    return dtype == KVA_F32 ? reinterpret_cast<const float *>(p)[i]
                            : bf16_bits_to_float(reinterpret_cast<const uint16_t *>(p)[i]);
}

__device__ inline void st_from_float(void *p, int dtype, size_t i, float v) {
    if (dtype == KVA_F32) reinterpret_cast<float *>(p)[i] = v;
    else reinterpret_cast<uint16_t *>(p)[i] = float_to_bf16_bits(v);
}

// One workgroup per output row.  x <- x + d1 + d2 (written back unless rows are gathered), then
// out_k = (x - mean) / sqrt(var + eps) * w_k with the variance as the mean of squared deviations.
// With rms != 0 the mean is not taken off: out_k = x / sqrt(mean(x^2) + eps) * w_k.
__global__ void __launch_bounds__(256)
layernorm_kernel(void *__restrict__ out1, void *__restrict__ out2, int out_dtype, void *__restrict__ x, int x_dtype,
                 const void *__restrict__ d1, int d1_dtype, const void *__restrict__ d2, int d2_dtype,
                 const void *__restrict__ w1, const void *__restrict__ w2, int w_dtype,
                 const int *__restrict__ row_idx, int width, float eps, int rms, float delta_scale) {
    extern __shared__ float row_s[];
    __shared__ float red_s[4];
    const int r = blockIdx.x;
    const size_t src = (size_t)(row_idx ? row_idx[r] : r) * width, dst = (size_t)r * width;
    float sum = 0.f;
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        float v = ld_as_float(x, x_dtype, src + j);
        if (delta_scale == 1.0f) {
            if (d1) v += ld_as_float(d1, d1_dtype, src + j);
            if (d2) v += ld_as_float(d2, d2_dtype, src + j);
        } else if (d1 || d2) {
            // the branch outputs are added up first, and their sum enters the stream times a constant
            const float b = (d1 ? ld_as_float(d1, d1_dtype, src + j) : 0.f) + (d2 ? ld_as_float(d2, d2_dtype, src + j) : 0.f);
            v += delta_scale * b;
        }
        if ((d1 || d2) && !row_idx) {
            st_from_float(x, x_dtype, src + j, v);
            v = ld_as_float(x, x_dtype, src + j);       // what the stream holds from now on
        } else if (d1 || d2) {
            if (x_dtype == KVA_BF16) v = bf16_bits_to_float(float_to_bf16_bits(v));
        }
        row_s[j] = v;
        sum += v;
    }
    float mean = 0.f;
    if (!rms) mean = block_sum(sum, red_s, blockDim.x / KVA_WAVE) / (float)width;
    float sq = 0.f;
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        const float dv = row_s[j] - mean;
        sq += dv * dv;
    }
    const float var = block_sum(sq, red_s, blockDim.x / KVA_WAVE) / (float)width;
    const float inv = 1.0f / sqrtf(var + eps);
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        const float n = (row_s[j] - mean) * inv;
        st_from_float(out1, out_dtype, dst + j, n * ld_as_float(w1, w_dtype, j));
        if (out2) st_from_float(out2, out_dtype, dst + j, n * ld_as_float(w2, w_dtype, j));
    }
}

extern "C" int kva_layernorm(void *out1, void *out2, int out_dtype, void *x, int x_dtype, const void *d1,
                             int d1_dtype, const void *d2, int d2_dtype, const void *w1, const void *w2,
                             int w_dtype, const int *row_idx, int rows, int width, float eps, int rms,
                             float delta_scale, hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && width > 0 && width <= 16000, "layernorm: width %d must lie in 1..16000", width);
    KVA_REQUIRE(out1 && x && w1 && (out2 == nullptr) == (w2 == nullptr), "layernorm: an output without its weight");
    KVA_REQUIRE(eps >= 0.f, "layernorm: negative eps");
    if (rows == 0) return KVA_OK;
    hipLaunchKernelGGL(layernorm_kernel, dim3(rows), dim3(256), (size_t)width * sizeof(float), stream, out1, out2,
                       out_dtype, x, x_dtype, d1, d1_dtype, d2, d2_dtype, w1, w2, w_dtype, row_idx, width, eps, rms, delta_scale);
    KVA_CHECK_LAUNCH("layernorm");
    return KVA_OK;
}

// out[t] = [ x[t] + d1[t] + d2[t] ; y[t] ] in out's type; x takes the sum (in place).
__global__ void stream_join_kernel(void *__restrict__ out, int out_dtype, void *__restrict__ x, int x_dtype,
                                   const void *__restrict__ d1, int d1_dtype, const void *__restrict__ d2,
                                   int d2_dtype, const void *__restrict__ y, int y_dtype, int wx, int wy) {
    const size_t t = blockIdx.x;
    for (int j = threadIdx.x; j < wx; j += blockDim.x) {
        float v = ld_as_float(x, x_dtype, t * wx + j);
        if (d1) v += ld_as_float(d1, d1_dtype, t * wx + j);
        if (d2) v += ld_as_float(d2, d2_dtype, t * wx + j);
        if (d1 || d2) {
            st_from_float(x, x_dtype, t * wx + j, v);
            v = ld_as_float(x, x_dtype, t * wx + j);
        }
        st_from_float(out, out_dtype, t * (wx + wy) + j, v);
    }
    for (int j = threadIdx.x; j < wy; j += blockDim.x)
        st_from_float(out, out_dtype, t * (wx + wy) + wx + j, ld_as_float(y, y_dtype, t * wy + j));
}

extern "C" int kva_stream_join(void *out, int out_dtype, void *x, int x_dtype, const void *d1, int d1_dtype,
                               const void *d2, int d2_dtype, const void *y, int y_dtype, int rows, int wx, int wy,
                               hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && wx > 0 && wy >= 0, "stream_join: bad sizes");
    KVA_REQUIRE(out && x && (wy == 0 || y), "stream_join: missing operand");
    if (rows == 0) return KVA_OK;
    hipLaunchKernelGGL(stream_join_kernel, dim3(rows), dim3(256), 0, stream, out, out_dtype, x, x_dtype, d1,
                       d1_dtype, d2, d2_dtype, y, y_dtype, wx, wy);
    KVA_CHECK_LAUNCH("stream_join");
    return KVA_OK;
}

// out[t, i] = act(gu[t, i]) * gu[t, inter + i]
__global__ void act_mul_kernel(void *__restrict__ out, const void *__restrict__ gu, int dtype, int inter, int act,
                               float limit) {
    const size_t t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= inter) return;
    const float g = ld_as_float(gu, dtype, t * 2 * inter + i), u = ld_as_float(gu, dtype, t * 2 * inter + inter + i);
    st_from_float(out, dtype, t * inter + i, kva_gated_activate(g, u, act, limit));
}

// bf16, inter a multiple of 8: a thread takes 8 neighbouring columns with 16-byte loads and stores
__global__ void act_mul_vec_kernel(uint4 *__restrict__ out, const uint4 *__restrict__ gu, int inter8, int act, float limit) {
    const size_t t = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= inter8) return;
    const uint4 gv = gu[t * 2 * inter8 + i], uv = gu[t * 2 * inter8 + inter8 + i];
    const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
    uint32_t ow[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float g0 = bf16_bits_to_float((uint16_t)(gw[j] & 0xffffu)), g1 = bf16_bits_to_float((uint16_t)(gw[j] >> 16));
        const float u0 = bf16_bits_to_float((uint16_t)(uw[j] & 0xffffu)), u1 = bf16_bits_to_float((uint16_t)(uw[j] >> 16));
        ow[j] = (uint32_t)float_to_bf16_bits(kva_gated_activate(g0, u0, act, limit)) |
                ((uint32_t)float_to_bf16_bits(kva_gated_activate(g1, u1, act, limit)) << 16);
    }
    out[t * inter8 + i] = make_uint4(ow[0], ow[1], ow[2], ow[3]);
}

extern "C" int kva_act_mul(void *out, const void *gate_up, int rows, int inter, int act, float limit, int dtype,
                           hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && rows <= 65535 && inter > 0, "act_mul: bad sizes");
    KVA_REQUIRE(act >= KVA_ACT_SILU && act <= KVA_ACT_SWISH_CLAMPED, "act_mul: unknown activation %d", act);
    if (rows == 0) return KVA_OK;
    if (dtype == KVA_BF16 && inter % 8 == 0) {
        hipLaunchKernelGGL(act_mul_vec_kernel, dim3((inter / 8 + 255) / 256, rows), dim3(256), 0, stream, (uint4 *)out,
                           (const uint4 *)gate_up, inter / 8, act, limit);
        KVA_CHECK_LAUNCH("act_mul");
        return KVA_OK;
    }
    hipLaunchKernelGGL(act_mul_kernel, dim3((inter + 255) / 256, rows), dim3(256), 0, stream, out, gate_up, dtype,
                       inter, act, limit);
    KVA_CHECK_LAUNCH("act_mul");
    return KVA_OK;
}

// x[t, h, :] *= sigmoid(g[t * g_stride + h]) for heads of head_dim elements
__global__ void head_gate_kernel(void *__restrict__ x, const void *__restrict__ g, int dtype, int heads, int head_dim,
                                 int g_stride) {
    const size_t t = blockIdx.x;
    for (int j = threadIdx.x; j < heads * head_dim; j += blockDim.x) {
        const float z = ld_as_float(g, dtype, t * g_stride + j / head_dim);
        const float s = 1.0f / (1.0f + expf(-z));
        const size_t at = t * heads * head_dim + j;
        st_from_float(x, dtype, at, ld_as_float(x, dtype, at) * s);
    }
}

extern "C" int kva_head_gate(void *x, const void *g, int rows, int heads, int head_dim, int g_stride, int dtype,
                             hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && heads > 0 && head_dim > 0 && g_stride >= heads, "head_gate: bad sizes");
    if (rows == 0) return KVA_OK;
    hipLaunchKernelGGL(head_gate_kernel, dim3(rows), dim3(256), 0, stream, x, g, dtype, heads, head_dim, g_stride);
    KVA_CHECK_LAUNCH("head_gate");
    return KVA_OK;
}

// ---- a branch output that is normed before it enters the stream --------------------------------
// x[t] += y[t] / sqrt(mean(y[t]^2) + eps) * w (an RMS norm on the branch's OUTPUT; the stream itself
// is read by the branches as it is).  With `copy` the new row of the stream is also written in a
// second type: what the next branch's products read.  One workgroup a row; the sum of squares is
// taken in a fixed order.
__global__ void __launch_bounds__(256)
norm_into_stream_kernel(void *__restrict__ x, int x_dtype, const void *__restrict__ y, int y_dtype,
                        const void *__restrict__ w, int w_dtype, void *__restrict__ copy, int copy_dtype, int width,
                        float eps) {
    extern __shared__ float row_s[];
    __shared__ float red_s[4];
    const size_t at = (size_t)blockIdx.x * width;
    float sq = 0.f;
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        const float v = ld_as_float(y, y_dtype, at + j);
        row_s[j] = v;
        sq += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red_s, blockDim.x / KVA_WAVE) / (float)width + eps);
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        const float v = ld_as_float(x, x_dtype, at + j) + row_s[j] * inv * ld_as_float(w, w_dtype, j);
        st_from_float(x, x_dtype, at + j, v);
        if (copy) st_from_float(copy, copy_dtype, at + j, x_dtype == KVA_F32 ? v : ld_as_float(x, x_dtype, at + j));
    }
}

// The same for the shapes a bf16 engine with a 32-bit stream has (x fp32, y bf16, copy bf16 or none, a
// width that is a multiple of 8 up to 2,048 * ITERS): a thread keeps its 8 * ITERS elements of y, x and w
// in registers, all loads are asked for before the sum of squares is taken, and rows move 16 bytes a
// lane.  At a few rows the launch is as long as its chain of trips to memory; this makes it one trip.
template <int ITERS>
__global__ void __launch_bounds__(256)
norm_into_stream_vec_kernel(float *__restrict__ x, const uint16_t *__restrict__ y, const void *__restrict__ w, int w_dtype,
                            uint16_t *__restrict__ copy, int width, float eps) {
    __shared__ float red_s[4];
    const size_t at = (size_t)blockIdx.x * width;
    float yv[ITERS][8], xv[ITERS][8], wv[ITERS][8];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (threadIdx.x + it * 256) * 8;
        if (j < width) {
            const uint4 yb = *reinterpret_cast<const uint4 *>(y + at + j);
            const float4 x0 = *reinterpret_cast<const float4 *>(x + at + j), x1 = *reinterpret_cast<const float4 *>(x + at + j + 4);
            const uint32_t yw[4] = {yb.x, yb.y, yb.z, yb.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                yv[it][2 * e] = __uint_as_float(yw[e] << 16);
                yv[it][2 * e + 1] = __uint_as_float(yw[e] & 0xffff0000u);
            }
            xv[it][0] = x0.x; xv[it][1] = x0.y; xv[it][2] = x0.z; xv[it][3] = x0.w;
            xv[it][4] = x1.x; xv[it][5] = x1.y; xv[it][6] = x1.z; xv[it][7] = x1.w;
            if (w_dtype == KVA_F32) {
                const float4 w0 = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(w) + j),
                             w1 = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(w) + j + 4);
                wv[it][0] = w0.x; wv[it][1] = w0.y; wv[it][2] = w0.z; wv[it][3] = w0.w;
                wv[it][4] = w1.x; wv[it][5] = w1.y; wv[it][6] = w1.z; wv[it][7] = w1.w;
            } else {
                const uint4 wb = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(w) + j);
                const uint32_t ww[4] = {wb.x, wb.y, wb.z, wb.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    wv[it][2 * e] = __uint_as_float(ww[e] << 16);
                    wv[it][2 * e + 1] = __uint_as_float(ww[e] & 0xffff0000u);
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) yv[it][e] = xv[it][e] = wv[it][e] = 0.f;
        }
    }
    float sq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += yv[it][e] * yv[it][e];
    const float inv = 1.0f / sqrtf(block_sum(sq, red_s, 4) / (float)width + eps);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (threadIdx.x + it * 256) * 8;
        if (j >= width) continue;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = xv[it][e] + yv[it][e] * inv * wv[it][e];
        *reinterpret_cast<float4 *>(x + at + j) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4 *>(x + at + j + 4) = make_float4(v[4], v[5], v[6], v[7]);
        if (copy) {
            uint32_t c[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                c[e] = (uint32_t)float_to_bf16_bits(v[2 * e]) | ((uint32_t)float_to_bf16_bits(v[2 * e + 1]) << 16);
            *reinterpret_cast<uint4 *>(copy + at + j) = make_uint4(c[0], c[1], c[2], c[3]);
        }
    }
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

extern "C" int kva_norm_into_stream(void *x, int x_dtype, const void *y, int y_dtype, const void *w, int w_dtype,
                                    void *copy, int copy_dtype, int rows, int width, float eps, hipStream_t stream) {
    KVA_REQUIRE(rows >= 0 && width > 0 && width <= 16000, "norm_into_stream: width %d must lie in 1..16000", width);
    KVA_REQUIRE(x && y && w && eps >= 0.f, "norm_into_stream: missing operand or negative eps");
    if (rows == 0) return KVA_OK;
    // (which kernel runs depends on types and width alone, never on the rows: a row's numbers are the same in any batch)
    if (x_dtype == KVA_F32 && y_dtype == KVA_BF16 && (!copy || copy_dtype == KVA_BF16) && width % 8 == 0 && width <= 8192 &&
        aligned16(x) && aligned16(y) && aligned16(w) && aligned16(copy)) {
        if (width <= 2048)
            hipLaunchKernelGGL(norm_into_stream_vec_kernel<1>, dim3(rows), dim3(256), 0, stream, (float *)x, (const uint16_t *)y,
                               w, w_dtype, (uint16_t *)copy, width, eps);
        else if (width <= 4096)
            hipLaunchKernelGGL(norm_into_stream_vec_kernel<2>, dim3(rows), dim3(256), 0, stream, (float *)x, (const uint16_t *)y,
                               w, w_dtype, (uint16_t *)copy, width, eps);
        else
            hipLaunchKernelGGL(norm_into_stream_vec_kernel<4>, dim3(rows), dim3(256), 0, stream, (float *)x, (const uint16_t *)y,
                               w, w_dtype, (uint16_t *)copy, width, eps);
        KVA_CHECK_LAUNCH("norm_into_stream");
        return KVA_OK;
    }
    hipLaunchKernelGGL(norm_into_stream_kernel, dim3(rows), dim3(256), (size_t)width * sizeof(float), stream, x, x_dtype,
                       y, y_dtype, w, w_dtype, copy, copy_dtype, width, eps);
    KVA_CHECK_LAUNCH("norm_into_stream");
    return KVA_OK;
}

// ---- a gate times a row of a table that the token picks ------------------------------------------
// out[t, j] = act(z[t, j]) * table[id_t, col0 + j] for j < dim: what a token brings of its own (a
// slice of a second embedding table) under a gate computed from the stream.  A negative id -1 - r
// stands for feedback[r], as in the embedding gather.
__global__ void __launch_bounds__(256)
table_gate_kernel(void *__restrict__ out, const void *__restrict__ z, int dtype, const void *__restrict__ table,
                  int table_dtype, int table_width, int table_rows, int col0, const int *__restrict__ ids,
                  const int *__restrict__ feedback, int dim, int act, int rows) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)rows * dim) return;
    const size_t t = i / dim;
    const int j = (int)(i % dim);
    int id = ids[t];
    if (id < 0) id = feedback[-1 - id];
    id = id < 0 ? 0 : (id >= table_rows ? table_rows - 1 : id);
    const float e = ld_as_float(table, table_dtype, (size_t)id * table_width + col0 + j);
    st_from_float(out, dtype, i, kva_activate(ld_as_float(z, dtype, i), act) * e);
}

extern "C" int kva_table_gate(void *out, const void *z, int dtype, const void *table, int table_dtype, int table_width,
                              int table_rows, int col0, const int *ids, const int *feedback, int rows, int dim, int act,
                              hipStream_t stream) {
    KVA_REQUIRE(out && z && table && ids && rows >= 0 && dim > 0 && table_rows > 0, "table_gate: missing operand or bad sizes");
    KVA_REQUIRE(col0 >= 0 && col0 + dim <= table_width, "table_gate: columns %d..%d lie outside a table row of %d", col0,
                col0 + dim, table_width);
    KVA_REQUIRE(act >= KVA_ACT_SILU && act <= KVA_ACT_GELU_TANH, "table_gate: unknown activation %d", act);
    if (rows == 0) return KVA_OK;
    const size_t n = (size_t)rows * dim;
    hipLaunchKernelGGL(table_gate_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, out, z, dtype, table,
                       table_dtype, table_width, table_rows, col0, ids, feedback, dim, act, rows);
    KVA_CHECK_LAUNCH("table_gate");
    return KVA_OK;
}

// ---- an activation over rows, with a bias ---------------------------------------------------------
// out[t, i] = act(x[t, i] + bias[i]) (the bias is optional): the middle of a feed-forward that is not gated.
__global__ void bias_act_kernel(void *__restrict__ out, const void *__restrict__ x, int dtype, const float *__restrict__ bias,
                                int width, int act, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = ld_as_float(x, dtype, i) + (bias ? bias[i % width] : 0.f);
    st_from_float(out, dtype, i, kva_activate(z, act));
}

extern "C" int kva_bias_act(void *out, const void *x, int dtype, const float *bias, int rows, int width, int act,
                            hipStream_t stream) {
    KVA_REQUIRE(out && x && rows >= 0 && width > 0, "bias_act: missing operand or bad sizes");
    KVA_REQUIRE(act >= KVA_ACT_SILU && act <= KVA_ACT_GELU_TANH, "bias_act: unknown activation %d", act);
    if (rows == 0) return KVA_OK;
    const size_t n = (size_t)rows * width;
    hipLaunchKernelGGL(bias_act_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, out, x, dtype, bias, width,
                       act, n);
    KVA_CHECK_LAUNCH("bias_act");
    return KVA_OK;
}

// ---- several copies of the stream (hyper-connections) -----------------------------------------------
// The residual stream is S copies x_1 .. x_S of every row, kept side by side: x [rows, S, width] fp32.
// One launch does what lies between two branches, a workgroup a row:
//   (1) with y, the branch output that is still to enter: all copies at once from the old ones,
//       x_t <- sum_s mix[s, t] x_s + mult * out_w[t] * y;
//   (2) with out: u = sum_s in_w[s] x_s of the new copies, then the layer norm with weight and bias,
//       out = (u - mean) / sqrt(var + eps) * w + b.
// With row_idx only the named rows are read (and nothing is written back): the model's last norm.
// S = 1 with mix = out_w = in_w = 1 is a plain residual stream whose branches enter times `mult`.
#define HYPER_MAX_STREAMS 8

struct HyperCoefficients {
    float mix[HYPER_MAX_STREAMS * HYPER_MAX_STREAMS], out_w[HYPER_MAX_STREAMS], in_w[HYPER_MAX_STREAMS];
};

template <int S>
__global__ void __launch_bounds__(256)
hyper_step_kernel(float *__restrict__ x, const void *__restrict__ y, int y_dtype, const float *__restrict__ mix,
                  const float *__restrict__ out_w, float mult, const float *__restrict__ in_w,
                  const void *__restrict__ nw, const void *__restrict__ nb, int w_dtype, float eps,
                  void *__restrict__ out, int out_dtype, const int *__restrict__ row_idx, int width) {
    extern __shared__ float row_s[];
    __shared__ float red_s[4];
    __shared__ HyperCoefficients co;
    const int r = blockIdx.x;
    const size_t row = (size_t)(row_idx ? row_idx[r] : r);
    if (threadIdx.x < S * S) co.mix[threadIdx.x] = y ? mix[threadIdx.x] : 0.f;
    if (threadIdx.x < S) {
        co.out_w[threadIdx.x] = y ? out_w[threadIdx.x] * mult : 0.f;
        co.in_w[threadIdx.x] = out ? in_w[threadIdx.x] : 0.f;
    }
    __syncthreads();
    float *xr = x + row * S * width;
    float sum = 0.f;
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        float v[S];
#pragma unroll
        for (int s = 0; s < S; ++s) v[s] = xr[(size_t)s * width + j];
        if (y) {
            const float yv = ld_as_float(y, y_dtype, row * width + j);
            float nv[S];
#pragma unroll
            for (int t = 0; t < S; ++t) {
                float acc = 0.f;
#pragma unroll
                for (int s = 0; s < S; ++s) acc += co.mix[s * S + t] * v[s];
                nv[t] = acc + co.out_w[t] * yv;
            }
#pragma unroll
            for (int t = 0; t < S; ++t) {
                v[t] = nv[t];
                if (!row_idx) xr[(size_t)t * width + j] = nv[t];
            }
        }
        if (out) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < S; ++s) u += co.in_w[s] * v[s];
            row_s[j] = u;
            sum += u;
        }
    }
    if (!out) return;
    const float mean = block_sum(sum, red_s, blockDim.x / KVA_WAVE) / (float)width;
    float sq = 0.f;
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        const float d = row_s[j] - mean;
        sq += d * d;
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red_s, blockDim.x / KVA_WAVE) / (float)width + eps);
    for (int j = threadIdx.x; j < width; j += blockDim.x)
        st_from_float(out, out_dtype, (size_t)r * width + j,
                      (row_s[j] - mean) * inv * ld_as_float(nw, w_dtype, j) + (nb ? ld_as_float(nb, w_dtype, j) : 0.f));
}

// The same with a row's elements in registers (a width that is a multiple of 4 up to 1,024 * ITERS, fp32 or
// bf16 operands): a thread takes 4 neighbouring columns ITERS times, asks for all its loads - the S copies,
// the branch output, the norm's weight and bias - before it uses any, and rows move 16 bytes a lane.  At a
// few rows the launch is as long as its chain of trips to memory; this makes it one trip.
__device__ inline void hyper_ld4(const void *p, int dtype, size_t i, float (&f)[4]) {
    if (dtype == KVA_F32) {
        const float4 v = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p) + i);
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
    } else {
        const uint2 v = *reinterpret_cast<const uint2 *>(reinterpret_cast<const uint16_t *>(p) + i);
        f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
        f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
    }
}

template <int S, int ITERS>
__global__ void __launch_bounds__(256)
hyper_step_vec_kernel(float *__restrict__ x, const void *__restrict__ y, int y_dtype, const float *__restrict__ mix,
                      const float *__restrict__ out_w, float mult, const float *__restrict__ in_w,
                      const void *__restrict__ nw, const void *__restrict__ nb, int w_dtype, float eps,
                      void *__restrict__ out, int out_dtype, const int *__restrict__ row_idx, int width) {
    __shared__ float red_s[4];
    __shared__ HyperCoefficients co;
    const int r = blockIdx.x;
    const size_t row = (size_t)(row_idx ? row_idx[r] : r);
    float *xr = x + row * S * width;
    float v[ITERS][S][4], yv[ITERS][4], wv[ITERS][4], bv[ITERS][4];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (threadIdx.x + it * 256) * 4;
        const bool on = j < width;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const float4 t = on ? *reinterpret_cast<const float4 *>(xr + (size_t)s * width + j) : make_float4(0.f, 0.f, 0.f, 0.f);
            v[it][s][0] = t.x; v[it][s][1] = t.y; v[it][s][2] = t.z; v[it][s][3] = t.w;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[it][e] = wv[it][e] = bv[it][e] = 0.f;
        if (on && y) hyper_ld4(y, y_dtype, row * width + j, yv[it]);
        if (on && out) hyper_ld4(nw, w_dtype, j, wv[it]);
        if (on && out && nb) hyper_ld4(nb, w_dtype, j, bv[it]);
    }
    if (threadIdx.x < S * S) co.mix[threadIdx.x] = y ? mix[threadIdx.x] : 0.f;
    if (threadIdx.x < S) {
        co.out_w[threadIdx.x] = y ? out_w[threadIdx.x] * mult : 0.f;
        co.in_w[threadIdx.x] = out ? in_w[threadIdx.x] : 0.f;
    }
    __syncthreads();
    float u[ITERS][4];
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (threadIdx.x + it * 256) * 4;
        const bool on = j < width;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (y) {
                float nv[S];
#pragma unroll
                for (int t = 0; t < S; ++t) {
                    float acc = 0.f;
#pragma unroll
                    for (int s = 0; s < S; ++s) acc += co.mix[s * S + t] * v[it][s][e];
                    nv[t] = acc + co.out_w[t] * yv[it][e];
                }
#pragma unroll
                for (int t = 0; t < S; ++t) v[it][t][e] = nv[t];
            }
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < S; ++s) a += co.in_w[s] * v[it][s][e];
            u[it][e] = on ? a : 0.f;
            sum += u[it][e];
        }
        if (y && !row_idx && on) {
#pragma unroll
            for (int t = 0; t < S; ++t)
                *reinterpret_cast<float4 *>(xr + (size_t)t * width + j) = make_float4(v[it][t][0], v[it][t][1], v[it][t][2], v[it][t][3]);
        }
    }
    if (!out) return;
    const float mean = block_sum(sum, red_s, 4) / (float)width;
    float sq = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const bool on = (threadIdx.x + it * 256) * 4 < width;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float d = on ? u[it][e] - mean : 0.f;
            sq += d * d;
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red_s, 4) / (float)width + eps);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int j = (threadIdx.x + it * 256) * 4;
        if (j >= width) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (u[it][e] - mean) * inv * wv[it][e] + bv[it][e];
        if (out_dtype == KVA_F32) {
            *reinterpret_cast<float4 *>(reinterpret_cast<float *>(out) + (size_t)r * width + j) = make_float4(o[0], o[1], o[2], o[3]);
        } else {
            *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(out) + (size_t)r * width + j) =
                make_uint2((uint32_t)float_to_bf16_bits(o[0]) | ((uint32_t)float_to_bf16_bits(o[1]) << 16),
                           (uint32_t)float_to_bf16_bits(o[2]) | ((uint32_t)float_to_bf16_bits(o[3]) << 16));
        }
    }
}

template <int S>
static bool hyper_step_vec(float *x, const void *y, int y_dtype, const float *mix, const float *out_w, float mult,
                           const float *in_w, const void *norm_w, const void *norm_b, int w_dtype, float eps, void *out,
                           int out_dtype, const int *row_idx, int rows, int width, hipStream_t stream) {
    // (which kernel runs depends on sizes and types alone, never on the rows: a row's numbers are the same in any batch)
    if (width % 4 || ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(norm_w) |
                       reinterpret_cast<uintptr_t>(norm_b) | reinterpret_cast<uintptr_t>(out)) & 15))
        return false;
#define KVA_HYPER_VEC(ITERS)                                                                                               \
    hipLaunchKernelGGL((hyper_step_vec_kernel<S, ITERS>), dim3(rows), dim3(256), 0, stream, x, y, y_dtype, mix, out_w, mult,  \
                       in_w, norm_w, norm_b, w_dtype, eps, out, out_dtype, row_idx, width)
    if (width <= 1024) KVA_HYPER_VEC(1);
    else if (width <= 2048 && S <= 8) KVA_HYPER_VEC(2);
    else if (width <= 4096 && S <= 4) KVA_HYPER_VEC(4);
    else if (width <= 8192 && S <= 2) KVA_HYPER_VEC(8);
    else return false;
#undef KVA_HYPER_VEC
    return true;
}

extern "C" int kva_hyper_step(float *x, int streams, const void *y, int y_dtype, const float *mix, const float *out_w,
                              float mult, const float *in_w, const void *norm_w, const void *norm_b, int w_dtype, float eps,
                              void *out, int out_dtype, const int *row_idx, int rows, int width, hipStream_t stream) {
    KVA_REQUIRE(x && rows >= 0 && width > 0 && width <= 16000, "hyper_step: width %d must lie in 1..16000", width);
    KVA_REQUIRE(streams >= 1 && streams <= HYPER_MAX_STREAMS, "hyper_step: %d copies of the stream (1..%d are built)", streams,
                HYPER_MAX_STREAMS);
    KVA_REQUIRE(!y || (mix && out_w), "hyper_step: a branch output enters through a mixing matrix and output weights");
    KVA_REQUIRE(!out || (in_w && norm_w && eps >= 0.f), "hyper_step: the read-out needs input weights and a norm");
    KVA_REQUIRE(y || out, "hyper_step: nothing to do");
    KVA_REQUIRE(!row_idx || out, "hyper_step: rows are gathered for the read-out only");
    if (rows == 0) return KVA_OK;
    bool done = false;
    switch (streams) {
        case 1: done = hyper_step_vec<1>(x, y, y_dtype, mix, out_w, mult, in_w, norm_w, norm_b, w_dtype, eps, out, out_dtype, row_idx, rows, width, stream); break;
        case 2: done = hyper_step_vec<2>(x, y, y_dtype, mix, out_w, mult, in_w, norm_w, norm_b, w_dtype, eps, out, out_dtype, row_idx, rows, width, stream); break;
        case 3: done = hyper_step_vec<3>(x, y, y_dtype, mix, out_w, mult, in_w, norm_w, norm_b, w_dtype, eps, out, out_dtype, row_idx, rows, width, stream); break;
        case 4: done = hyper_step_vec<4>(x, y, y_dtype, mix, out_w, mult, in_w, norm_w, norm_b, w_dtype, eps, out, out_dtype, row_idx, rows, width, stream); break;
        default: break;
    }
    if (done) {
        KVA_CHECK_LAUNCH("hyper_step");
        return KVA_OK;
    }
    const size_t lds = (size_t)width * sizeof(float);
#define KVA_HYPER_CASE(S)                                                                                               \
    case S:                                                                                                             \
        hipLaunchKernelGGL(hyper_step_kernel<S>, dim3(rows), dim3(256), lds, stream, x, y, y_dtype, mix, out_w, mult, in_w,  \
                           norm_w, norm_b, w_dtype, eps, out, out_dtype, row_idx, width);                              \
        break;
    switch (streams) {
        KVA_HYPER_CASE(1) KVA_HYPER_CASE(2) KVA_HYPER_CASE(3) KVA_HYPER_CASE(4)
        KVA_HYPER_CASE(5) KVA_HYPER_CASE(6) KVA_HYPER_CASE(7) KVA_HYPER_CASE(8)
    }
#undef KVA_HYPER_CASE
    KVA_CHECK_LAUNCH("hyper_step");
    return KVA_OK;
}

// every row of `first` [rows, width] (any storage type) into all S copies of x [rows, S, width] fp32: the
// stream as the embedding leaves it
__global__ void hyper_fill_kernel(float *__restrict__ x, const void *__restrict__ first, int dtype, int streams, int width,
                                  size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / width, j = i % width;
    const float v = ld_as_float(first, dtype, i);
    for (int s = 0; s < streams; ++s) x[(t * streams + s) * width + j] = v;
}

extern "C" int kva_hyper_fill(float *x, const void *first, int dtype, int streams, int rows, int width, hipStream_t stream) {
    KVA_REQUIRE(x && first && streams >= 1 && rows >= 0 && width > 0, "hyper_fill: missing operand or bad sizes");
    if (rows == 0) return KVA_OK;
    const size_t n = (size_t)rows * width;
    hipLaunchKernelGGL(hyper_fill_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, first, dtype, streams,
                       width, n);
    KVA_CHECK_LAUNCH("hyper_fill");
    return KVA_OK;
}
