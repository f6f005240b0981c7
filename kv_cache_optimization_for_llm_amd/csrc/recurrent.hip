// Mixers that carry a fixed-size state per request instead of keys and values:
//
//  * kva_causal_conv_act / kva_conv_state_update: a short causal convolution over time per channel
//    followed by silu; the last taps - 1 inputs of a request are part of its state.
//  * kva_gated_delta_rule: per head S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with
//    unit-norm q and k, one decay g = exp(-exp(A_log) softplus(a + dt_bias)) per head and token - or a
//    decay per head and key channel, handed in ready-made, that multiplies the rows of S one by one.
//  * kva_gated_linear_attention: per head S <- diag(alpha) S + k v^T; o = S^T q with a decay per
//    key channel, alpha = sigmoid(z)^(1 / tau) - or one fixed decay a head for all channels and tokens;
//    q, k and v may pass an activation (silu) on their way in.
//  * kva_head_norm_gate: every head of a row divided by its root mean square (optional) times a
//    weight, times act(gate), times a constant, into a column range of a wider buffer.
//
// The state S [key channels, value channels] of a (request, head) is fp32 and lives in the seat's
// state row between steps.  Columns are independent of each other in both recurrences, so a head's
// columns go to different wavefronts, which walk the step's tokens of the request in order.  Key sizes
// up to 128 keep their part of S in registers (4 columns a wavefront, 16 lanes a column); larger
// ones keep it in LDS (16 columns a wavefront, lane = 16 r + c owns the rows r, r + 4, ... of column
// c).  The order of every sum depends on the sizes alone: a token's result is the same bit for bit
// however the request's tokens were cut into steps and whatever else the step holds.
#include "common.h"
#include <math.h>

#define REC_COLS 16          // value columns a wavefront takes
#define REC_ROWGROUPS 4      // lanes that share a column
#define REC_MAX_DIM 512

__device__ inline float rec_ld(const void *p, int dtype, size_t i) {
    return dtype == KVA_BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(p)[i])
                             : reinterpret_cast<const float *>(p)[i];
}

__device__ inline void rec_st(void *p, int dtype, size_t i, float v) {
    if (dtype == KVA_BF16) reinterpret_cast<uint16_t *>(p)[i] = float_to_bf16_bits(v);
    else reinterpret_cast<float *>(p)[i] = v;
}

__device__ inline float rec_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
__device__ inline float rec_silu(float z) { return z / (1.f + expf(-z)); }
__device__ inline float rec_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ inline float rec_act(float z, int act) { return act == 1 ? rec_silu(z) : z; }

// sum over the lanes that share a column (lanes c, c + 16, c + 32, c + 48), all of them get it
__device__ inline float rec_column_sum(float v) {
    v += __shfl_xor(v, 16, KVA_WAVE);
    v += __shfl_xor(v, 32, KVA_WAVE);
    return v;
}

// ---- short causal convolution + silu -----------------------------------------------------
// out[row, c] = act(sum_j w[c, j] * in(row - taps + 1 + j)[c] + out_bias[c]) with act = silu or none and
// in = y + in_bias (both biases optional); inputs before the step's first
// token of the request come from the seat's state [channels, taps - 1] (slot taps - 2 newest).
__global__ void __launch_bounds__(256)
causal_conv_act_kernel(float *__restrict__ out, int out_stride, const void *__restrict__ y, int y_dtype, int y_stride,
                       int col_off, const void *__restrict__ w, int w_dtype, const float *__restrict__ state,
                       size_t seat_stride, int conv_off, const int *__restrict__ entry_q_start,
                       const int *__restrict__ entry_seat, int channels, int taps, int tokens_per_block,
                       const float *__restrict__ in_bias, const float *__restrict__ out_bias, int act) {
    const int e = blockIdx.y;
    const int q0 = entry_q_start[e], n = entry_q_start[e + 1] - q0;
    const int first = blockIdx.x * tokens_per_block;
    if (first >= n) return;
    const int last = min(n, first + tokens_per_block);
    const float *st = state + (size_t)entry_seat[e] * seat_stride + conv_off;
    for (int c = threadIdx.x; c < channels; c += blockDim.x) {
        for (int i = first; i < last; ++i) {
            float acc = 0.f;
            for (int j = 0; j < taps; ++j) {
                const int src = i - (taps - 1) + j;
                // (the state holds inputs with their bias already added; before a request's start it holds zeros)
                const float x = src >= 0 ? rec_ld(y, y_dtype, (size_t)(q0 + src) * y_stride + col_off + c) + (in_bias ? in_bias[c] : 0.f)
                                         : st[(size_t)c * (taps - 1) + (taps - 1) + src];
                acc += rec_ld(w, w_dtype, (size_t)c * taps + j) * x;
            }
            if (out_bias) acc += out_bias[c];
            out[(size_t)(q0 + i) * out_stride + c] = rec_act(acc, act);
        }
    }
}

// the seat's last taps - 1 inputs after this step; a thread owns a channel (reads all, then writes)
__global__ void __launch_bounds__(256)
conv_state_update_kernel(float *__restrict__ state, size_t seat_stride, int conv_off, const void *__restrict__ y,
                         int y_dtype, int y_stride, int col_off, const int *__restrict__ entry_q_start,
                         const int *__restrict__ entry_seat, int channels, int taps, const float *__restrict__ in_bias) {
    const int e = blockIdx.y;
    const int q0 = entry_q_start[e], n = entry_q_start[e + 1] - q0;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels || n <= 0) return;
    float *st = state + (size_t)entry_seat[e] * seat_stride + conv_off + (size_t)c * (taps - 1);
    float keep[16];
    for (int s = 0; s < taps - 1; ++s) {
        const int src = n - (taps - 1) + s;
        keep[s] = src >= 0 ? rec_ld(y, y_dtype, (size_t)(q0 + src) * y_stride + col_off + c) + (in_bias ? in_bias[c] : 0.f) : st[s + n];
    }
    for (int s = 0; s < taps - 1; ++s) st[s] = keep[s];
}

extern "C" int kva_causal_conv_act(float *out, int out_stride, const void *y, int y_dtype, int y_stride, int col_off,
                                   const void *w, int w_dtype, float *state, long long seat_stride, int conv_off,
                                   const int *entry_q_start, const int *entry_seat, int entries, int max_q_len,
                                   int channels, int taps, const float *in_bias, const float *out_bias, int act,
                                   hipStream_t stream) {
    KVA_REQUIRE(act == 0 || act == 1, "causal_conv_act: activation %d is neither none (0) nor silu (1)", act);
    KVA_REQUIRE(out && y && w && state && entry_q_start && entry_seat, "causal_conv_act: missing operand");
    KVA_REQUIRE(channels > 0 && taps >= 1 && taps <= 17, "causal_conv_act: taps %d must lie in 1..17", taps);
    KVA_REQUIRE(entries >= 0 && entries <= 65535 && max_q_len >= 0, "causal_conv_act: bad batch");
    if (entries == 0 || max_q_len == 0) return KVA_OK;
    const int per = 8;
    hipLaunchKernelGGL(causal_conv_act_kernel, dim3((max_q_len + per - 1) / per, entries), dim3(256), 0, stream, out,
                       out_stride, y, y_dtype, y_stride, col_off, w, w_dtype, state, (size_t)seat_stride, conv_off,
                       entry_q_start, entry_seat, channels, taps, per, in_bias, out_bias, act);
    KVA_CHECK_LAUNCH("causal_conv_act");
    if (taps > 1) {
        hipLaunchKernelGGL(conv_state_update_kernel, dim3((channels + 255) / 256, entries), dim3(256), 0, stream, state,
                           (size_t)seat_stride, conv_off, y, y_dtype, y_stride, col_off, entry_q_start, entry_seat,
                           channels, taps, in_bias);
        KVA_CHECK_LAUNCH("conv_state_update");
    }
    return KVA_OK;
}

// ---- the two recurrences -----------------------------------------------------------------
// LDS: S [dim][16] fp32, then per chunk of tokens q [chunk][dim], k [chunk][dim], (alpha [chunk][dim]),
// and per token two numbers.
struct RecArgs {
    float *out;                 // [T, heads * vdim] fp32
    float *state;               // seat rows; this mixer's S [heads, dim, vdim] at state_off
    size_t seat_stride;
    int state_off;
    const int *entry_q_start, *entry_seat;
    int heads, kv_heads, dim, vdim, chunk;
};

// Gated delta rule.  q, k, v are the convolution's fp32 output rows [T, conv_stride]: q at
// column 0 (kv_heads x dim), k behind it, v behind that (heads x vdim).  beta and the decay's input
// are columns of the projection y.
__global__ void __launch_bounds__(KVA_WAVE)
gated_delta_rule_kernel(RecArgs a, const float *__restrict__ qkv, int conv_stride, const void *__restrict__ y,
                        int y_dtype, int y_stride, int beta_off, int decay_off, const float *__restrict__ a_log,
                        const float *__restrict__ dt_bias, float unit_eps, const float *__restrict__ channel_decay,
                        int decay_stride) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x, c = lane % REC_COLS, r = lane / REC_COLS;
    const int slices = (a.vdim + REC_COLS - 1) / REC_COLS;
    const int head = blockIdx.x / slices, col = (blockIdx.x % slices) * REC_COLS + c;
    const int e = blockIdx.y;
    const int q0 = a.entry_q_start[e], n = a.entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int d = a.dim, dv = a.vdim, kvh = head / (a.heads / a.kv_heads);
    const bool on = col < dv;
    float *S = lds, *qs = S + d * REC_COLS, *ks = qs + a.chunk * d, *bs = ks + a.chunk * d, *gs = bs + a.chunk;
    float *as = gs + a.chunk;            // with a decay per key channel: the chunk's decays [chunk][dim]
    float *Sg = a.state + (size_t)a.entry_seat[e] * a.seat_stride + a.state_off + (size_t)head * d * dv;
    for (int i = r; i < d; i += REC_ROWGROUPS) S[i * REC_COLS + c] = on ? Sg[(size_t)i * dv + col] : 0.f;
    const int k_col = a.kv_heads * d, v_col = 2 * a.kv_heads * d;
    const float rate = channel_decay ? 0.f : expf(a_log[head]), bias = channel_decay ? 0.f : dt_bias[head];
    const float q_mul = 1.0f / sqrtf((float)d);
    for (int t0 = 0; t0 < n; t0 += a.chunk) {
        const int m = min(a.chunk, n - t0);
        __syncthreads();
        for (int x = lane; x < m * d; x += KVA_WAVE) {
            const size_t row = (size_t)(q0 + t0 + x / d) * conv_stride;
            qs[x] = qkv[row + kvh * d + x % d];
            ks[x] = qkv[row + k_col + kvh * d + x % d];
            if (channel_decay) as[x] = channel_decay[(size_t)(q0 + t0 + x / d) * decay_stride + head * d + x % d];
        }
        __syncthreads();
        // unit vectors: token tt by the four lanes 4 tt .. 4 tt + 3 (chunk <= 16)
        {
            const int tt = lane / 4, part = lane % 4;
            float sq = 0.f, sk = 0.f;
            if (tt < m)
                for (int i = part; i < d; i += 4) {
                    sq += qs[tt * d + i] * qs[tt * d + i];
                    sk += ks[tt * d + i] * ks[tt * d + i];
                }
            sq += __shfl_xor(sq, 1, KVA_WAVE); sq += __shfl_xor(sq, 2, KVA_WAVE);
            sk += __shfl_xor(sk, 1, KVA_WAVE); sk += __shfl_xor(sk, 2, KVA_WAVE);
            const float mq = q_mul / sqrtf(sq + unit_eps), mk = 1.0f / sqrtf(sk + unit_eps);
            __syncthreads();
            if (tt < m) {
                for (int i = part; i < d; i += 4) {
                    qs[tt * d + i] *= mq;
                    ks[tt * d + i] *= mk;
                }
                if (part == 0) {
                    const size_t yrow = (size_t)(q0 + t0 + tt) * y_stride;
                    bs[tt] = rec_sigmoid(rec_ld(y, y_dtype, yrow + beta_off + head));
                    gs[tt] = channel_decay ? 1.f : expf(-rate * rec_softplus(rec_ld(y, y_dtype, yrow + decay_off + head) + bias));
                }
            }
        }
        __syncthreads();
        for (int tt = 0; tt < m; ++tt) {
            const float *q = qs + tt * d, *k = ks + tt * d;
            const float g = gs[tt], beta = bs[tt];
            const size_t row = (size_t)(q0 + t0 + tt);
            const float v = on ? qkv[row * conv_stride + v_col + head * dv + col] : 0.f;
            float dot = 0.f;
            if (channel_decay) {      // the rows of S are decayed one by one before S^T k is taken
                const float *al = as + tt * d;
                for (int i = r; i < d; i += REC_ROWGROUPS) S[i * REC_COLS + c] *= al[i];
            }
            for (int i = r; i < d; i += REC_ROWGROUPS) dot += S[i * REC_COLS + c] * k[i];
            dot = rec_column_sum(dot);
            const float u = beta * (v - g * dot);
            float o = 0.f;
            for (int i = r; i < d; i += REC_ROWGROUPS) {
                const float s = g * S[i * REC_COLS + c] + k[i] * u;
                S[i * REC_COLS + c] = s;
                o += s * q[i];
            }
            o = rec_column_sum(o);
            if (on && r == 0) a.out[row * a.heads * dv + head * dv + col] = o;
        }
    }
    if (on)
        for (int i = r; i < d; i += REC_ROWGROUPS) Sg[(size_t)i * dv + col] = S[i * REC_COLS + c];
}

// Gated linear attention.  q, k, v are columns of y (heads x dim, heads x dim, heads x vdim); the
// decays alpha (heads x dim a token, fp32) come in a buffer of their own; q is multiplied by q_mul.
__global__ void __launch_bounds__(KVA_WAVE)
gated_linear_attention_kernel(RecArgs a, const void *__restrict__ y, int y_dtype, int y_stride, int q_off, int k_off,
                              int v_off, const float *__restrict__ alpha, int alpha_stride, float q_mul,
                              const float *__restrict__ head_decay, int act) {
    extern __shared__ float lds[];
    const int lane = threadIdx.x, c = lane % REC_COLS, r = lane / REC_COLS;
    const int slices = (a.vdim + REC_COLS - 1) / REC_COLS;
    const int head = blockIdx.x / slices, col = (blockIdx.x % slices) * REC_COLS + c;
    const int e = blockIdx.y;
    const int q0 = a.entry_q_start[e], n = a.entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int d = a.dim, dv = a.vdim;
    const bool on = col < dv;
    float *S = lds, *qs = S + d * REC_COLS, *ks = qs + a.chunk * d, *as = ks + a.chunk * d;
    float *Sg = a.state + (size_t)a.entry_seat[e] * a.seat_stride + a.state_off + (size_t)head * d * dv;
    for (int i = r; i < d; i += REC_ROWGROUPS) S[i * REC_COLS + c] = on ? Sg[(size_t)i * dv + col] : 0.f;
    for (int t0 = 0; t0 < n; t0 += a.chunk) {
        const int m = min(a.chunk, n - t0);
        __syncthreads();
        for (int x = lane; x < m * d; x += KVA_WAVE) {
            const size_t row = (size_t)(q0 + t0 + x / d);
            const int i = head * d + x % d;
            qs[x] = rec_act(rec_ld(y, y_dtype, row * y_stride + q_off + i), act) * q_mul;
            ks[x] = rec_act(rec_ld(y, y_dtype, row * y_stride + k_off + i), act);
            as[x] = alpha ? alpha[row * alpha_stride + i] : head_decay[head];
        }
        __syncthreads();
        for (int tt = 0; tt < m; ++tt) {
            const float *q = qs + tt * d, *k = ks + tt * d, *al = as + tt * d;
            const size_t row = (size_t)(q0 + t0 + tt);
            const float v = on ? rec_act(rec_ld(y, y_dtype, row * y_stride + v_off + head * dv + col), act) : 0.f;
            float o = 0.f;
            for (int i = r; i < d; i += REC_ROWGROUPS) {
                const float s = al[i] * S[i * REC_COLS + c] + k[i] * v;
                S[i * REC_COLS + c] = s;
                o += s * q[i];
            }
            o = rec_column_sum(o);
            if (on && r == 0) a.out[row * a.heads * dv + head * dv + col] = o;
        }
    }
    if (on)
        for (int i = r; i < d; i += REC_ROWGROUPS) Sg[(size_t)i * dv + col] = S[i * REC_COLS + c];
}

// ---- the two recurrences with the state in registers (key sizes up to 128) ----------------------
// A workgroup of four wavefronts takes 16 value columns of a head, a wavefront 4 of them; the 16
// lanes of a row of the wavefront share a column.  Lane (c, r) owns, of column c, the rows
// 4 (16 j + r) .. + 3 for j < RP / 4 in RP registers (rows from `dim` on are padding and stay zero): a
// 16-byte LDS read per j and lane takes 256 neighbouring bytes of a token's k, q or alpha, and a sum
// over the rows ends with four rotations inside the lanes' row.  A chunk of 32 tokens is staged in
// LDS once for the four wavefronts - q, k (and the decays) padded to 16 RP elements a token, the 16
// values of the workgroup's columns, the token's numbers; the next chunk's global loads are issued
// before the current one is walked, and no wavefront waits for another inside a chunk.
#define REC_CHUNK 32         // tokens staged at a time: their walk hides the next chunk's trip to memory
#define REG_COLS 4           // columns a wavefront
#define REG_LANES 16         // lanes that share a column
#define REG_WAVES 4
#define REG_BLOCK_COLS (REG_COLS * REG_WAVES)
#define REG_THREADS (KVA_WAVE * REG_WAVES)

// Sums over the 16 lanes of a row for several values at once, stage by stage: the rotations of one
// value do not wait for each other's results but stand between those of the others (a dependent
// instruction of a wavefront that has its SIMD to itself waits some 16 cycles for its operand).
template <int N>
__device__ inline void row16_sum_each(float (&x)[N]) {
    float t[N];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = row16_rotated<8>(x[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] += t[i];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = row16_rotated<4>(x[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] += t[i];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = row16_rotated<2>(x[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] += t[i];
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = row16_rotated<1>(x[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) x[i] += t[i];
}

// CD: the decay has one value per head and key channel and comes ready-made, fp32 [T, heads * dim]
// (`channel_decay`); the rows of S are then decayed one by one and the head's single decay is not formed.
template <int RP, bool CD>
__global__ void __launch_bounds__(REG_THREADS)
gated_delta_rule_reg_kernel(RecArgs a, const float *__restrict__ qkv, int conv_stride, const void *__restrict__ y,
                            int y_dtype, int y_stride, int beta_off, int decay_off, const float *__restrict__ a_log,
                            const float *__restrict__ dt_bias, float unit_eps, const float *__restrict__ channel_decay,
                            int decay_stride) {
    constexpr int DP = REG_LANES * RP, DS = DP + 4, CH = REC_CHUNK, PER = CH * DP / REG_THREADS;   // token rows 4 banks apart
    __shared__ __attribute__((aligned(16))) float qs[CH * DS];
    __shared__ __attribute__((aligned(16))) float ks[CH * DS];
    __shared__ __attribute__((aligned(16))) float as[CD ? CH * DS : 4];
    __shared__ float vs[CH * REG_BLOCK_COLS], os[CH * REG_BLOCK_COLS], bs[CH], gs[CH], nq[CH], nk[CH];
    const int tid = threadIdx.x, lane = tid % KVA_WAVE, wave = tid / KVA_WAVE;
    const int c = lane / REG_LANES, r = lane % REG_LANES;
    const int slices = (a.vdim + REG_BLOCK_COLS - 1) / REG_BLOCK_COLS;
    const int head = blockIdx.x / slices, block_col0 = (blockIdx.x % slices) * REG_BLOCK_COLS;
    const int col = block_col0 + wave * REG_COLS + c;
    const int e = blockIdx.y;
    const int q0 = a.entry_q_start[e], n = a.entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int d = a.dim, dv = a.vdim, kvh = head / (a.heads / a.kv_heads);
    const bool on = col < dv;
    float *Sg = a.state + (size_t)a.entry_seat[e] * a.seat_stride + a.state_off + (size_t)head * d * dv;
    float S[RP];
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int i = 4 * (REG_LANES * (j / 4) + r) + j % 4;
        S[j] = (on && i < d) ? Sg[(size_t)i * dv + col] : 0.f;
    }
    const int k_col = a.kv_heads * d, v_col = 2 * a.kv_heads * d;
    const float rate = CD ? 0.f : expf(a_log[head]), bias = CD ? 0.f : dt_bias[head], q_mul = 1.0f / sqrtf((float)d);
    constexpr int VPER = CH * REG_BLOCK_COLS / REG_THREADS;
    float pq[PER], pk[PER], pa[CD ? PER : 1], pv[VPER], pb = 0.f, pg = 0.f;
    auto fetch = [&](int t0, int m) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            pq[j] = pk[j] = 0.f;
            if constexpr (CD) pa[j] = 0.f;
            if (REG_THREADS * j / DP >= m) continue;        // (the whole workgroup: a decoded token loads one row)
            const int x = tid + REG_THREADS * j, tt = x / DP, i = x % DP;
            if (tt >= m || i >= d) continue;
            const size_t row = (size_t)(q0 + t0 + tt) * conv_stride;
            pq[j] = qkv[row + kvh * d + i];
            pk[j] = qkv[row + k_col + kvh * d + i];
            if constexpr (CD) pa[j] = channel_decay[(size_t)(q0 + t0 + tt) * decay_stride + head * d + i];
        }
#pragma unroll
        for (int j = 0; j < VPER; ++j) {   // the chunk's tokens x 16 columns
            const int x = tid + REG_THREADS * j, tt = x / REG_BLOCK_COLS, cc = x % REG_BLOCK_COLS;
            pv[j] = (tt < m && block_col0 + cc < dv)
                        ? qkv[(size_t)(q0 + t0 + tt) * conv_stride + v_col + head * dv + block_col0 + cc] : 0.f;
        }
        if (tid < m) {
            const size_t yrow = (size_t)(q0 + t0 + tid) * y_stride;
            pb = rec_ld(y, y_dtype, yrow + beta_off + head);
            if constexpr (!CD) pg = rec_ld(y, y_dtype, yrow + decay_off + head);
        }
    };
    fetch(0, min(CH, n));
    for (int t0 = 0; t0 < n; t0 += CH) {
        const int m = min(CH, n - t0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int x = tid + REG_THREADS * j, at = (x / DP) * DS + x % DP;
            qs[at] = pq[j];
            ks[at] = pk[j];
            if constexpr (CD) as[at] = pa[j];
        }
#pragma unroll
        for (int j = 0; j < VPER; ++j) vs[tid + REG_THREADS * j] = pv[j];
        if (tid < m) {
            bs[tid] = rec_sigmoid(pb);
            gs[tid] = CD ? 1.f : expf(-rate * rec_softplus(pg + bias));
        }
        __syncthreads();
        if (wave < CH / 16) {   // what makes q and k unit vectors: a token by four lanes, every fourth element each
            const int tt = wave * 16 + lane / 4, part = lane % 4;
            float sq = 0.f, sk = 0.f;
            if (tt < m)
                for (int i = part; i < DP; i += 4) {
                    sq += qs[tt * DS + i] * qs[tt * DS + i];
                    sk += ks[tt * DS + i] * ks[tt * DS + i];
                }
            sq += __shfl_xor(sq, 1, KVA_WAVE); sq += __shfl_xor(sq, 2, KVA_WAVE);
            sk += __shfl_xor(sk, 1, KVA_WAVE); sk += __shfl_xor(sk, 2, KVA_WAVE);
            if (part == 0) {
                nq[tt] = q_mul / sqrtf(sq + unit_eps);
                nk[tt] = 1.0f / sqrtf(sk + unit_eps);
            }
        }
        __syncthreads();
        if (t0 + CH < n) fetch(t0 + CH, min(CH, n - t0 - CH));
        // The walk.  Both sums over the rows that a token needs read the same S - the state before the
        // token for S^T k, the state after it for S^T q - so the read-out of a token rides with the next
        // token's S^T k: one pass over S, the two sums reduced side by side, and only the chain
        // S^T k -> u -> S is what a token waits for.
        float4 qp[RP / 4];                       // q of the token before (zero in front of the chunk's first)
        float mqp = 0.f;
#pragma unroll
        for (int j = 0; j < RP / 4; ++j) qp[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int tt = 0; tt <= m; ++tt) {
            const bool last = tt == m;           // behind the chunk's last token only its read-out is left
            const int at = min(tt, CH - 1);
            const float4 *k4 = reinterpret_cast<const float4 *>(ks + at * DS) + r;
            const float4 *q4 = reinterpret_cast<const float4 *>(qs + at * DS) + r;
            const float g = gs[at], beta = bs[at], v = vs[at * REG_BLOCK_COLS + wave * REG_COLS + c], mq = nq[at], mk = nk[at];
            float4 kk[RP / 4], qq[RP / 4];
            float Sd[CD ? RP : 1];               // the decayed rows, where every row has a decay of its own
            float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f, p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
            for (int j = 0; j < RP / 4; ++j) {
                kk[j] = k4[REG_LANES * j];
                qq[j] = q4[REG_LANES * j];
                // the unit vectors' factors multiply the sums: S^T (mk k) = mk (S^T k), S^T (mq q) likewise
                kk[j].x *= mk; kk[j].y *= mk; kk[j].z *= mk; kk[j].w *= mk;
                if constexpr (CD) {
                    const float4 al = (reinterpret_cast<const float4 *>(as + at * DS) + r)[REG_LANES * j];
                    Sd[4 * j] = al.x * S[4 * j];
                    Sd[4 * j + 1] = al.y * S[4 * j + 1];
                    Sd[4 * j + 2] = al.z * S[4 * j + 2];
                    Sd[4 * j + 3] = al.w * S[4 * j + 3];
                    d0 += Sd[4 * j] * kk[j].x;
                    d1 += Sd[4 * j + 1] * kk[j].y;
                    d2 += Sd[4 * j + 2] * kk[j].z;
                    d3 += Sd[4 * j + 3] * kk[j].w;
                } else {
                    d0 += S[4 * j] * kk[j].x;
                    d1 += S[4 * j + 1] * kk[j].y;
                    d2 += S[4 * j + 2] * kk[j].z;
                    d3 += S[4 * j + 3] * kk[j].w;
                }
                p0 += S[4 * j] * qp[j].x;
                p1 += S[4 * j + 1] * qp[j].y;
                p2 += S[4 * j + 2] * qp[j].z;
                p3 += S[4 * j + 3] * qp[j].w;
            }
            d0 += d1; p0 += p1; d2 += d3; p2 += p3;
            float both[2] = {d0 + d2, p0 + p2};
            row16_sum_each<2>(both);
            if (tt > 0 && r == 0) os[(tt - 1) * REG_BLOCK_COLS + wave * REG_COLS + c] = both[1] * mqp;
            if (last) break;
            const float u = beta * (v - g * both[0]);
#pragma unroll
            for (int j = 0; j < RP / 4; ++j) {
                if constexpr (CD) {
                    S[4 * j] = Sd[4 * j] + kk[j].x * u;
                    S[4 * j + 1] = Sd[4 * j + 1] + kk[j].y * u;
                    S[4 * j + 2] = Sd[4 * j + 2] + kk[j].z * u;
                    S[4 * j + 3] = Sd[4 * j + 3] + kk[j].w * u;
                } else {
                    S[4 * j] = g * S[4 * j] + kk[j].x * u;
                    S[4 * j + 1] = g * S[4 * j + 1] + kk[j].y * u;
                    S[4 * j + 2] = g * S[4 * j + 2] + kk[j].z * u;
                    S[4 * j + 3] = g * S[4 * j + 3] + kk[j].w * u;
                }
                qp[j] = qq[j];
            }
            mqp = mq;
        }
        __syncthreads();
        // the chunk's read-outs leave together, 16 neighbouring columns a token
#pragma unroll
        for (int j = 0; j < VPER; ++j) {
            const int x = tid + REG_THREADS * j, tt = x / REG_BLOCK_COLS, cc = x % REG_BLOCK_COLS;
            if (tt < m && block_col0 + cc < dv)
                a.out[(size_t)(q0 + t0 + tt) * a.heads * dv + head * dv + block_col0 + cc] = os[x];
        }
    }
    if (on)
#pragma unroll
        for (int j = 0; j < RP; ++j) {
            const int i = 4 * (REG_LANES * (j / 4) + r) + j % 4;
            if (i < d) Sg[(size_t)i * dv + col] = S[j];
        }
}

template <int RP>
__global__ void __launch_bounds__(REG_THREADS)
gated_linear_attention_reg_kernel(RecArgs a, const void *__restrict__ y, int y_dtype, int y_stride, int q_off, int k_off,
                                  int v_off, const float *__restrict__ alpha, int alpha_stride, float q_mul,
                                  const float *__restrict__ head_decay, int act) {
    constexpr int DP = REG_LANES * RP, DS = DP + 4, CH = REC_CHUNK, PER = CH * DP / REG_THREADS;   // token rows 4 banks apart
    __shared__ __attribute__((aligned(16))) float qs[CH * DS];
    __shared__ __attribute__((aligned(16))) float ks[CH * DS];
    __shared__ __attribute__((aligned(16))) float as[CH * DS];
    __shared__ float vs[CH * REG_BLOCK_COLS], os[CH * REG_BLOCK_COLS];
    const int tid = threadIdx.x, lane = tid % KVA_WAVE, wave = tid / KVA_WAVE;
    const int c = lane / REG_LANES, r = lane % REG_LANES;
    const int slices = (a.vdim + REG_BLOCK_COLS - 1) / REG_BLOCK_COLS;
    const int head = blockIdx.x / slices, block_col0 = (blockIdx.x % slices) * REG_BLOCK_COLS;
    const int col = block_col0 + wave * REG_COLS + c;
    const int e = blockIdx.y;
    const int q0 = a.entry_q_start[e], n = a.entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int d = a.dim, dv = a.vdim;
    const bool on = col < dv;
    float *Sg = a.state + (size_t)a.entry_seat[e] * a.seat_stride + a.state_off + (size_t)head * d * dv;
    float S[RP];
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int i = 4 * (REG_LANES * (j / 4) + r) + j % 4;
        S[j] = (on && i < d) ? Sg[(size_t)i * dv + col] : 0.f;
    }
    constexpr int VPER = CH * REG_BLOCK_COLS / REG_THREADS;
    float pq[PER], pk[PER], pa[PER], pv[VPER];
    const float fixed = alpha ? 0.f : head_decay[head];     // one decay for the head's every channel and token
    auto fetch = [&](int t0, int m) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            pq[j] = pk[j] = pa[j] = 0.f;
            if (REG_THREADS * j / DP >= m) continue;        // (the whole workgroup: a decoded token loads one row)
            const int x = tid + REG_THREADS * j, tt = x / DP, i = x % DP;
            if (tt >= m || i >= d) continue;
            const size_t row = (size_t)(q0 + t0 + tt);
            pq[j] = rec_act(rec_ld(y, y_dtype, row * y_stride + q_off + head * d + i), act);
            pk[j] = rec_act(rec_ld(y, y_dtype, row * y_stride + k_off + head * d + i), act);
            pa[j] = alpha ? alpha[row * alpha_stride + head * d + i] : fixed;
        }
#pragma unroll
        for (int j = 0; j < VPER; ++j) {   // the chunk's tokens x 16 columns
            const int x = tid + REG_THREADS * j, tt = x / REG_BLOCK_COLS, cc = x % REG_BLOCK_COLS;
            pv[j] = (tt < m && block_col0 + cc < dv)
                        ? rec_act(rec_ld(y, y_dtype, (size_t)(q0 + t0 + tt) * y_stride + v_off + head * dv + block_col0 + cc), act) : 0.f;
        }
    };
    fetch(0, min(CH, n));
    for (int t0 = 0; t0 < n; t0 += CH) {
        const int m = min(CH, n - t0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int x = tid + REG_THREADS * j, at = (x / DP) * DS + x % DP;
            qs[at] = pq[j] * q_mul;
            ks[at] = pk[j];
            as[at] = pa[j];
        }
#pragma unroll
        for (int j = 0; j < VPER; ++j) vs[tid + REG_THREADS * j] = pv[j];
        __syncthreads();
        if (t0 + CH < n) fetch(t0 + CH, min(CH, n - t0 - CH));
        // The walk, four tokens at a time: only S is handed from token to token (two operations an
        // element); the four read-outs' sums over the rows are independent of each other and are
        // formed side by side, stage by stage.
        auto step = [&](int tt, float (&o)[4]) {
            const float4 *k4 = reinterpret_cast<const float4 *>(ks + tt * DS) + r;
            const float4 *q4 = reinterpret_cast<const float4 *>(qs + tt * DS) + r;
            const float4 *a4 = reinterpret_cast<const float4 *>(as + tt * DS) + r;
            const float v = vs[tt * REG_BLOCK_COLS + wave * REG_COLS + c];
            o[0] = o[1] = o[2] = o[3] = 0.f;
#pragma unroll
            for (int j = 0; j < RP / 4; ++j) {
                const float4 kk = k4[REG_LANES * j], qq = q4[REG_LANES * j], al = a4[REG_LANES * j];
                S[4 * j] = al.x * S[4 * j] + kk.x * v;
                S[4 * j + 1] = al.y * S[4 * j + 1] + kk.y * v;
                S[4 * j + 2] = al.z * S[4 * j + 2] + kk.z * v;
                S[4 * j + 3] = al.w * S[4 * j + 3] + kk.w * v;
                o[0] += S[4 * j] * qq.x;
                o[1] += S[4 * j + 1] * qq.y;
                o[2] += S[4 * j + 2] * qq.z;
                o[3] += S[4 * j + 3] * qq.w;
            }
        };
        int tt = 0;
        for (; tt + 4 <= m; tt += 4) {
            float o[4][4], sum[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) step(tt + i, o[i]);
#pragma unroll
            for (int i = 0; i < 4; ++i) { o[i][0] += o[i][1]; o[i][2] += o[i][3]; }
#pragma unroll
            for (int i = 0; i < 4; ++i) sum[i] = o[i][0] + o[i][2];
            row16_sum_each<4>(sum);
            if (r == 0)
#pragma unroll
                for (int i = 0; i < 4; ++i) os[(tt + i) * REG_BLOCK_COLS + wave * REG_COLS + c] = sum[i];
        }
        for (; tt < m; ++tt) {
            float o[4];
            step(tt, o);
            const float sum = row16_sum((o[0] + o[1]) + (o[2] + o[3]));
            if (r == 0) os[tt * REG_BLOCK_COLS + wave * REG_COLS + c] = sum;
        }
        __syncthreads();
        // the chunk's read-outs leave together, 16 neighbouring columns a token
#pragma unroll
        for (int j = 0; j < VPER; ++j) {
            const int x = tid + REG_THREADS * j, tt = x / REG_BLOCK_COLS, cc = x % REG_BLOCK_COLS;
            if (tt < m && block_col0 + cc < dv)
                a.out[(size_t)(q0 + t0 + tt) * a.heads * dv + head * dv + block_col0 + cc] = os[x];
        }
    }
    if (on)
#pragma unroll
        for (int j = 0; j < RP; ++j) {
            const int i = 4 * (REG_LANES * (j / 4) + r) + j % 4;
            if (i < d) Sg[(size_t)i * dv + col] = S[j];
        }
}

static int rec_chunk(int dim, int arrays) {
    // tokens staged at a time: 16 where the LDS has room for them beside the state, else 4
    const size_t room = 60 * 1024;
    for (int chunk = 16; chunk >= 4; chunk /= 4)
        if (((size_t)dim * REC_COLS + (size_t)chunk * dim * arrays + 2 * chunk) * sizeof(float) <= room) return chunk;
    return 0;
}

static int rec_check(const char *what, const void *out, const void *state, const int *q_start, const int *seat,
                     int entries, int heads, int kv_heads, int dim, int vdim) {
    KVA_REQUIRE(out && state && q_start && seat, "%s: missing operand", what);
    KVA_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "%s: %d heads over %d key heads", what, heads, kv_heads);
    KVA_REQUIRE(dim > 0 && dim <= REC_MAX_DIM && vdim > 0, "%s: key size %d must lie in 1..%d", what, dim, REC_MAX_DIM);
    KVA_REQUIRE(entries >= 0 && entries <= 65535, "%s: %d entries", what, entries);
    return KVA_OK;
}

extern "C" int kva_gated_delta_rule(float *out, float *state, long long seat_stride, int state_off, const float *qkv,
                                    int conv_stride, const void *y, int y_dtype, int y_stride, int beta_off,
                                    int decay_off, const float *a_log, const float *dt_bias, float unit_eps,
                                    const float *channel_decay, int decay_stride,
                                    const int *entry_q_start, const int *entry_seat, int entries, int heads,
                                    int kv_heads, int dim, int vdim, hipStream_t stream) {
    if (int rc = rec_check("gated_delta_rule", out, state, entry_q_start, entry_seat, entries, heads, kv_heads, dim, vdim)) return rc;
    // the decay: one per head, formed here from a column of y, a rate and a bias - or one per head and
    // key channel, handed in ready-made (fp32 [T, >= heads * dim])
    KVA_REQUIRE(qkv && y && ((a_log && dt_bias) || (channel_decay && decay_stride >= heads * dim)),
                "gated_delta_rule: missing operand");
    if (entries == 0) return KVA_OK;
    if (dim <= 128) {
        RecArgs a{out, state, (size_t)seat_stride, state_off, entry_q_start, entry_seat, heads, kv_heads, dim, vdim, REC_CHUNK};
        const dim3 grid(heads * ((vdim + REG_BLOCK_COLS - 1) / REG_BLOCK_COLS), entries);
#define KVA_DELTA_REG(RP)                                                                                              \
    do {                                                                                                               \
        if (channel_decay)                                                                                             \
            hipLaunchKernelGGL((gated_delta_rule_reg_kernel<RP, true>), grid, dim3(REG_THREADS), 0, stream, a, qkv,      \
                               conv_stride, y, y_dtype, y_stride, beta_off, decay_off, a_log, dt_bias, unit_eps,      \
                               channel_decay, decay_stride);                                                           \
        else                                                                                                           \
            hipLaunchKernelGGL((gated_delta_rule_reg_kernel<RP, false>), grid, dim3(REG_THREADS), 0, stream, a, qkv,     \
                               conv_stride, y, y_dtype, y_stride, beta_off, decay_off, a_log, dt_bias, unit_eps,      \
                               channel_decay, decay_stride);                                                           \
    } while (0)
        if (dim <= 64) KVA_DELTA_REG(4);
        else KVA_DELTA_REG(8);
#undef KVA_DELTA_REG
        KVA_CHECK_LAUNCH("gated_delta_rule");
        return KVA_OK;
    }
    const int arrays = channel_decay ? 3 : 2;
    const int chunk = rec_chunk(dim, arrays);
    KVA_REQUIRE(chunk > 0, "gated_delta_rule: key size %d does not fit the LDS", dim);
    RecArgs a{out, state, (size_t)seat_stride, state_off, entry_q_start, entry_seat, heads, kv_heads, dim, vdim, chunk};
    const size_t lds = ((size_t)dim * REC_COLS + (size_t)chunk * dim * arrays + 2 * chunk) * sizeof(float);
    const int slices = (vdim + REC_COLS - 1) / REC_COLS;
    hipLaunchKernelGGL(gated_delta_rule_kernel, dim3(heads * slices, entries), dim3(KVA_WAVE), lds, stream, a, qkv,
                       conv_stride, y, y_dtype, y_stride, beta_off, decay_off, a_log, dt_bias, unit_eps, channel_decay,
                       decay_stride);
    KVA_CHECK_LAUNCH("gated_delta_rule");
    return KVA_OK;
}

extern "C" int kva_gated_linear_attention(float *out, float *state, long long seat_stride, int state_off,
                                          const void *y, int y_dtype, int y_stride, int q_off, int k_off, int v_off,
                                          const float *alpha, int alpha_stride, float q_mul,
                                          const float *head_decay, int act,
                                          const int *entry_q_start, const int *entry_seat,
                                          int entries, int heads, int dim, int vdim, hipStream_t stream) {
    if (int rc = rec_check("gated_linear_attention", out, state, entry_q_start, entry_seat, entries, heads, heads, dim, vdim)) return rc;
    // the decays: a buffer with one value per token, head and key channel, or one fixed value a head
    KVA_REQUIRE(y && ((alpha && alpha_stride >= heads * dim) || (!alpha && head_decay)), "gated_linear_attention: missing operand");
    KVA_REQUIRE(act == 0 || act == 1, "gated_linear_attention: activation %d is neither none (0) nor silu (1)", act);
    if (entries == 0) return KVA_OK;
    if (dim <= 128) {
        RecArgs a{out, state, (size_t)seat_stride, state_off, entry_q_start, entry_seat, heads, heads, dim, vdim, REC_CHUNK};
        const dim3 grid(heads * ((vdim + REG_BLOCK_COLS - 1) / REG_BLOCK_COLS), entries);
#define KVA_GLA_REG(RP)                                                                                                \
    hipLaunchKernelGGL(gated_linear_attention_reg_kernel<RP>, grid, dim3(REG_THREADS), 0, stream, a, y, y_dtype,          \
                       y_stride, q_off, k_off, v_off, alpha, alpha_stride, q_mul, head_decay, act)
        if (dim <= 64) KVA_GLA_REG(4);
        else KVA_GLA_REG(8);
#undef KVA_GLA_REG
        KVA_CHECK_LAUNCH("gated_linear_attention");
        return KVA_OK;
    }
    const int chunk = rec_chunk(dim, 3);
    KVA_REQUIRE(chunk > 0, "gated_linear_attention: key size %d does not fit the LDS", dim);
    RecArgs a{out, state, (size_t)seat_stride, state_off, entry_q_start, entry_seat, heads, heads, dim, vdim, chunk};
    const size_t lds = ((size_t)dim * REC_COLS + (size_t)chunk * dim * 3) * sizeof(float);
    const int slices = (vdim + REC_COLS - 1) / REC_COLS;
    hipLaunchKernelGGL(gated_linear_attention_kernel, dim3(heads * slices, entries), dim3(KVA_WAVE), lds, stream, a, y,
                       y_dtype, y_stride, q_off, k_off, v_off, alpha, alpha_stride, q_mul, head_decay, act);
    KVA_CHECK_LAUNCH("gated_linear_attention");
    return KVA_OK;
}

// ---- per-head norm and gate ----------------------------------------------------------------
// out[t, out_off + h dv + j] = (x[t, h, j] / sqrt(mean_j x^2 + eps) * w[j], or x as it is without a
// weight) * act(gate[t, gate_off + h dv + j]) * mul;  act: 0 silu, 1 sigmoid.  One wavefront a head.
__global__ void __launch_bounds__(256)
head_norm_gate_kernel(void *__restrict__ out, int out_dtype, int out_stride, int out_off, const void *__restrict__ x,
                      int x_dtype, const float *__restrict__ w, float eps, const void *__restrict__ gate,
                      int gate_dtype, int gate_stride, int gate_off, int heads, int dv, int act, float mul, int w_stride) {
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE, waves = blockDim.x / KVA_WAVE;
    for (int h = wave; h < heads; h += waves) {
        const size_t base = (t * heads + h) * dv;
        float inv = 1.f;
        if (w) {
            float sq = 0.f;
            for (int j = lane; j < dv; j += KVA_WAVE) {
                const float v = rec_ld(x, x_dtype, base + j);
                sq += v * v;
            }
            inv = 1.0f / sqrtf(wave_sum(sq) / (float)dv + eps);
        }
        for (int j = lane; j < dv; j += KVA_WAVE) {
            float v = rec_ld(x, x_dtype, base + j);
            if (w) v = v * inv * w[(size_t)h * w_stride + j];
            if (gate) {
                const float g = rec_ld(gate, gate_dtype, t * gate_stride + gate_off + h * dv + j);
                v *= (act == 1 ? rec_sigmoid(g) : rec_silu(g));
            }
            v *= mul;
            rec_st(out, out_dtype, t * out_stride + out_off + h * dv + j, v);
        }
    }
}

// Few wide heads (one norm over a whole row, say): the workgroup takes the heads one after the other,
// all its wavefronts on each; the sum of squares is taken in a fixed order.
__global__ void __launch_bounds__(256)
head_norm_gate_wide_kernel(void *__restrict__ out, int out_dtype, int out_stride, int out_off, const void *__restrict__ x,
                           int x_dtype, const float *__restrict__ w, float eps, const void *__restrict__ gate,
                           int gate_dtype, int gate_stride, int gate_off, int heads, int dv, int act, float mul, int w_stride) {
    __shared__ float red_s[4];
    const size_t t = blockIdx.x;
    for (int h = 0; h < heads; ++h) {
        const size_t base = (t * heads + h) * dv;
        float inv = 1.f;
        if (w) {
            float sq = 0.f;
            for (int j = threadIdx.x; j < dv; j += blockDim.x) {
                const float v = rec_ld(x, x_dtype, base + j);
                sq += v * v;
            }
            inv = 1.0f / sqrtf(block_sum(sq, red_s, blockDim.x / KVA_WAVE) / (float)dv + eps);
        }
        for (int j = threadIdx.x; j < dv; j += blockDim.x) {
            float v = rec_ld(x, x_dtype, base + j);
            if (w) v = v * inv * w[(size_t)h * w_stride + j];
            if (gate) {
                const float g = rec_ld(gate, gate_dtype, t * gate_stride + gate_off + h * dv + j);
                v *= (act == 1 ? rec_sigmoid(g) : rec_silu(g));
            }
            v *= mul;
            rec_st(out, out_dtype, t * out_stride + out_off + h * dv + j, v);
        }
    }
}

extern "C" int kva_head_norm_gate(void *out, int out_dtype, int out_stride, int out_off, const void *x, int x_dtype,
                                  const float *w, float eps, const void *gate, int gate_dtype, int gate_stride,
                                  int gate_off, int rows, int heads, int dv, int act, float mul, int w_stride,
                                  hipStream_t stream) {
    // w_stride: 0 - one weight of dv elements shared by the heads; dv - a weight of heads * dv elements.  gate may be absent.
    KVA_REQUIRE(out && x && heads > 0 && dv > 0 && rows >= 0, "head_norm_gate: missing operand or bad sizes");
    KVA_REQUIRE(w_stride == 0 || w_stride == dv, "head_norm_gate: a weight is shared by the heads or has all heads' size");
    KVA_REQUIRE(act == 0 || act == 1, "head_norm_gate: activation %d is neither silu (0) nor sigmoid (1)", act);
    if (rows == 0) return KVA_OK;
    if (heads < 4 && dv >= 256)
        hipLaunchKernelGGL(head_norm_gate_wide_kernel, dim3(rows), dim3(256), 0, stream, out, out_dtype, out_stride, out_off,
                           x, x_dtype, w, eps, gate, gate_dtype, gate_stride, gate_off, heads, dv, act, mul, w_stride);
    else
        hipLaunchKernelGGL(head_norm_gate_kernel, dim3(rows), dim3(256), 0, stream, out, out_dtype, out_stride, out_off, x,
                           x_dtype, w, eps, gate, gate_dtype, gate_stride, gate_off, heads, dv, act, mul, w_stride);
    KVA_CHECK_LAUNCH("head_norm_gate");
    return KVA_OK;
}

// ---- a real-gated linear recurrent unit ------------------------------------------------------------
// Channels come in `blocks` equal runs; inside run b two square matrices [out, in] make the gates from
// the run's own inputs u_b: r = sigmoid(A_b u_b + a_b), i = sigmoid(B_b u_b + b_b).  The recurrence
// S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with log a_t = -rate_c r_t (rate_c = 8 softplus(lam_c), formed
// once when the weights are loaded) is linear in S, so this kernel forms, for all tokens side by side,
// a_t and the input b_t = sqrt(1 - a_t^2) i_t u_t, and kva_linear_scan_gate walks the tokens.
// A workgroup takes 64 tokens x 64 outputs of one run, a thread 4 x 4 of them for both matrices (operands
// through LDS, 16 inputs at a time).  k ascending into one accumulator per output: a token's numbers do not
// depend on the batch.
#define BG_BM 64
#define BG_BN 64
#define BG_BK 16
__global__ void __launch_bounds__(256)
block_gates_kernel(float *__restrict__ a_out, float *__restrict__ b_out, const float *__restrict__ u, int tokens, int width,
                   int bs, const void *__restrict__ wa, const void *__restrict__ wi, int w_dtype,
                   const float *__restrict__ ba, const float *__restrict__ bi, const float *__restrict__ rate) {
    __shared__ float Us[BG_BK][BG_BM + 4], Was[BG_BK][BG_BN + 4], Wis[BG_BK][BG_BN + 4];
    const int blk = blockIdx.y, t0 = blockIdx.z * BG_BM, n0 = blockIdx.x * BG_BN;
    const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const size_t wbase = (size_t)blk * bs * bs;
    float ar[4][4], ai[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) ar[i][j] = ai[i][j] = 0.f;
    for (int k0 = 0; k0 < bs; k0 += BG_BK) {
        float xa[4], xr[4], xi[4];
        const int tok = t0 + lrow, wn = n0 + lrow;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int kk = k0 + lk + e;
            xa[e] = (tok < tokens && kk < bs) ? u[(size_t)tok * width + blk * bs + kk] : 0.f;
            const bool in = wn < bs && kk < bs;
            xr[e] = in ? rec_ld(wa, w_dtype, wbase + (size_t)wn * bs + kk) : 0.f;
            xi[e] = in ? rec_ld(wi, w_dtype, wbase + (size_t)wn * bs + kk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Us[lk + e][lrow] = xa[e];
            Was[lk + e][lrow] = xr[e];
            Wis[lk + e][lrow] = xi[e];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BG_BK; ++kk) {
            float uv[4], rv[4], iv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uv[i] = Us[kk][4 * ty + i];
                rv[i] = Was[kk][4 * tx + i];
                iv[i] = Wis[kk][4 * tx + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    ar[i][j] += uv[i] * rv[j];
                    ai[i][j] += uv[i] * iv[j];
                }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = t0 + 4 * ty + i;
        if (t >= tokens) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + 4 * tx + j;
            if (n >= bs) continue;
            const int c = blk * bs + n;
            const float r = rec_sigmoid(ar[i][j] + ba[c]), g = rec_sigmoid(ai[i][j] + bi[c]);
            const float log_a = -rate[c] * r;
            const size_t at = (size_t)t * width + c;
            a_out[at] = expf(log_a);
            b_out[at] = sqrtf(-expm1f(2.f * log_a)) * g * u[at];          // sqrt(1 - a^2) without the cancellation near a = 1
        }
    }
}

// Few tokens (decoding): a workgroup takes a token and 64 channels; the token's inputs go to LDS once, a
// wavefront takes 16 channels, four at a time with 16 lanes a channel: the lanes stride over the run's inputs
// (bf16 matrices with runs that are multiples of 8: 16 bytes a lane and load), all loads of the four rounds
// are independent of each other, and the 16 lanes add up by rotations inside their row of lanes.
__global__ void __launch_bounds__(256)
block_gates_rows_kernel(float *__restrict__ a_out, float *__restrict__ b_out, const float *__restrict__ u, int width, int bs,
                        const void *__restrict__ wa, const void *__restrict__ wi, int w_dtype,
                        const float *__restrict__ ba, const float *__restrict__ bi, const float *__restrict__ rate) {
    extern __shared__ float us[];
    const size_t t = blockIdx.x;
    const int c_lo = blockIdx.y * 64;
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE, r16 = lane % 16, sub = lane / 16;
    // (the inputs of the runs this workgroup's channels lie in)
    const int k_lo = (c_lo / bs) * bs, k_hi = min(width, ((min(c_lo + 64, width) - 1) / bs + 1) * bs);
    for (int k = k_lo + threadIdx.x; k < k_hi; k += blockDim.x) us[k - k_lo] = u[t * width + k];
    __syncthreads();
    const bool vec = w_dtype == KVA_BF16 && bs % 8 == 0;
    float ar[4], ai[4];
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        const int c = c_lo + 16 * wave + 4 * round + sub;
        ar[round] = ai[round] = 0.f;
        if (c >= width) continue;
        const int blk = c / bs;
        const size_t wrow = (size_t)blk * bs * bs + (size_t)(c - blk * bs) * bs;
        const float *xs = us + (blk * bs - k_lo);
        if (vec) {
            for (int k = 8 * r16; k < bs; k += 128) {
                const uint4 va = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(wa) + wrow + k);
                const uint4 vi = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(wi) + wrow + k);
                const uint32_t pa[4] = {va.x, va.y, va.z, va.w}, pi[4] = {vi.x, vi.y, vi.z, vi.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ar[round] += xs[k + 2 * e] * __uint_as_float(pa[e] << 16) + xs[k + 2 * e + 1] * __uint_as_float(pa[e] & 0xffff0000u);
                    ai[round] += xs[k + 2 * e] * __uint_as_float(pi[e] << 16) + xs[k + 2 * e + 1] * __uint_as_float(pi[e] & 0xffff0000u);
                }
            }
        } else {
            for (int k = r16; k < bs; k += 16) {
                ar[round] += xs[k] * rec_ld(wa, w_dtype, wrow + k);
                ai[round] += xs[k] * rec_ld(wi, w_dtype, wrow + k);
            }
        }
    }
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        const int c = c_lo + 16 * wave + 4 * round + sub;
        const float sr = row16_sum(ar[round]), si = row16_sum(ai[round]);
        if (r16 == 0 && c < width) {
            const float r = rec_sigmoid(sr + ba[c]), g = rec_sigmoid(si + bi[c]);
            const float log_a = -rate[c] * r;
            a_out[t * width + c] = expf(log_a);
            b_out[t * width + c] = sqrtf(-expm1f(2.f * log_a)) * g * us[c - k_lo];
        }
    }
}

extern "C" int kva_block_gates(float *a_out, float *b_out, const float *u, int tokens, int width, int blocks, const void *wa,
                               const void *wi, int w_dtype, const float *ba, const float *bi, const float *rate,
                               hipStream_t stream) {
    KVA_REQUIRE(a_out && b_out && u && wa && wi && ba && bi && rate, "block_gates: missing operand");
    KVA_REQUIRE(tokens >= 0 && width > 0 && blocks > 0 && width % blocks == 0, "block_gates: %d channels in %d equal runs", width, blocks);
    KVA_REQUIRE(w_dtype == KVA_BF16 || w_dtype == KVA_F32, "block_gates: unsupported dtype");
    if (tokens == 0) return KVA_OK;
    const int bs = width / blocks;
    if (tokens <= 32 && (width + 63) / 64 <= 65535) {
        // the inputs of at most 64 + 2 (bs - 1) channels' runs
        const size_t lds = (size_t)(bs >= 64 ? ((63 / bs) + 2) * bs : 64 + 2 * bs) * sizeof(float);
        if (lds <= 64 * 1024) {
            hipLaunchKernelGGL(block_gates_rows_kernel, dim3(tokens, (width + 63) / 64), dim3(256), lds, stream, a_out, b_out, u,
                               width, bs, wa, wi, w_dtype, ba, bi, rate);
            KVA_CHECK_LAUNCH("block_gates");
            return KVA_OK;
        }
    }
    KVA_REQUIRE(blocks <= 65535 && (tokens + BG_BM - 1) / BG_BM <= 65535, "block_gates: too many runs or tokens for one launch");
    hipLaunchKernelGGL(block_gates_kernel, dim3((bs + BG_BN - 1) / BG_BN, blocks, (tokens + BG_BM - 1) / BG_BM), dim3(256), 0, stream, a_out, b_out,
                       u, tokens, width, bs, wa, wi, w_dtype, ba, bi, rate);
    KVA_CHECK_LAUNCH("block_gates");
    return KVA_OK;
}

// S_t = a_t S_(t-1) + b_t per channel over each entry's tokens in order, from the seat's S [width] (which takes
// the last S_t); out[t, out_off + c] = S_t * act(gate[t, gate_off + c] + gate_bias[c]) * mul with act the tanh
// form of gelu.  The recurrence is linear, so a workgroup of 16 segments x 16 channels cuts an entry's
// tokens into 16 runs: every thread first folds its run into (A, B) with S_out = A S_in + B, the runs are
// chained in order through LDS, and a second walk over the run writes the results.
#define SCAN_SEGMENTS 16
#define SCAN_CHANNELS 16
__global__ void __launch_bounds__(256)
linear_scan_gate_kernel(void *__restrict__ out, int out_dtype, int out_stride, int out_off, const float *__restrict__ a,
                        const float *__restrict__ b, int width, const void *__restrict__ gate, int gate_dtype,
                        int gate_stride, int gate_off, const float *__restrict__ gate_bias, float *__restrict__ state,
                        size_t seat_stride, int state_off, const int *__restrict__ entry_q_start,
                        const int *__restrict__ entry_seat, float mul) {
    __shared__ float As[SCAN_SEGMENTS][SCAN_CHANNELS], Bs[SCAN_SEGMENTS][SCAN_CHANNELS];
    const int e = blockIdx.y;
    const int q0 = entry_q_start[e], n = entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int cl = threadIdx.x % SCAN_CHANNELS, seg = threadIdx.x / SCAN_CHANNELS;
    const int c = blockIdx.x * SCAN_CHANNELS + cl;
    const bool on = c < width;
    const int per = (n + SCAN_SEGMENTS - 1) / SCAN_SEGMENTS;
    const int lo = min(n, seg * per), hi = min(n, lo + per);
    float A = 1.f, B = 0.f;
    if (on)
        for (int i = lo; i < hi; ++i) {
            const size_t at = (size_t)(q0 + i) * width + c;
            const float av = a[at];
            A *= av;
            B = av * B + b[at];
        }
    As[seg][cl] = A;
    Bs[seg][cl] = B;
    __syncthreads();
    if (!on) return;
    float *st = state + (size_t)entry_seat[e] * seat_stride + state_off + c;
    float S = *st;
    for (int s2 = 0; s2 < seg; ++s2) S = As[s2][cl] * S + Bs[s2][cl];
    const float gb = gate_bias ? gate_bias[c] : 0.f;
    for (int i = lo; i < hi; ++i) {
        const size_t at = (size_t)(q0 + i) * width + c;
        S = a[at] * S + b[at];
        const float g = rec_ld(gate, gate_dtype, (size_t)(q0 + i) * gate_stride + gate_off + c) + gb;
        const float act = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
        rec_st(out, out_dtype, (size_t)(q0 + i) * out_stride + out_off + c, S * act * mul);
    }
    // the last segment's S is the entry's last state (an empty last segment holds it as its start)
    if (seg == SCAN_SEGMENTS - 1) *st = S;
}

extern "C" int kva_linear_scan_gate(void *out, int out_dtype, int out_stride, int out_off, const float *a, const float *b,
                                    int width, const void *gate, int gate_dtype, int gate_stride, int gate_off,
                                    const float *gate_bias, float *state, long long seat_stride, int state_off,
                                    const int *entry_q_start, const int *entry_seat, int entries, float mul,
                                    hipStream_t stream) {
    KVA_REQUIRE(out && a && b && gate && state && entry_q_start && entry_seat, "linear_scan_gate: missing operand");
    KVA_REQUIRE(width > 0 && entries >= 0 && entries <= 65535, "linear_scan_gate: bad sizes");
    if (entries == 0) return KVA_OK;
    hipLaunchKernelGGL(linear_scan_gate_kernel, dim3((width + SCAN_CHANNELS - 1) / SCAN_CHANNELS, entries), dim3(256), 0, stream,
                       out, out_dtype, out_stride, out_off, a, b, width, gate, gate_dtype, gate_stride, gate_off, gate_bias,
                       state, (size_t)seat_stride, state_off, entry_q_start, entry_seat, mul);
    KVA_CHECK_LAUNCH("linear_scan_gate");
    return KVA_OK;
}

// ---- a matrix memory with exponential gates -----------------------------------------------------------
// Per head a matrix S [dim, vdim], a vector n [dim] and a running maximum m (all zero at a request's start).
// With the token's log input gate i = cap tanh(zi / cap), log forget gate f = logsigmoid(cap tanh(zf / cap)):
//   m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n <- e^(f + m - m') n + e^(i - m') k;
//   o = S^T q / (max(|n . q|, e^(-m')) + 1e-6),  q times q_mul.
// zi, zf come as fp32 rows [T, 2 heads] (input gates first).  One wavefront takes 16 value columns of a head:
// lane = 16 r + c owns rows r, r + 4, ... of column c of S in LDS, and a copy of its rows of n; tokens are
// staged 16 at a time.  The seat's state row holds S [heads, dim, vdim], then n and then m once per
// wavefront, [heads, ceil(vdim / 16), dim] and [heads, ceil(vdim / 16)]: kva_matrix_memory_state says how much.
#define MM_STAGE 16
__global__ void __launch_bounds__(KVA_WAVE)
matrix_memory_kernel(float *__restrict__ out, float *__restrict__ state, size_t seat_stride, int state_off,
                     const void *__restrict__ y, int y_dtype, int y_stride, int q_off, int k_off, int v_off,
                     const float *__restrict__ gates, float cap, float q_mul, const int *__restrict__ entry_q_start,
                     const int *__restrict__ entry_seat, int heads, int dim, int vdim) {
    extern __shared__ float lds[];
    const int e = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * REC_COLS;
    const int q0 = entry_q_start[e], n = entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int lane = threadIdx.x, c = lane % REC_COLS, rg = lane / REC_COLS;
    const int col = col0 + c;
    const bool col_on = col < vdim;
    float *S = lds;                                   // [dim][16]
    float *N = S + (size_t)dim * REC_COLS;            // [dim][16]: every column's lanes keep their own copy
    float *qs = N + (size_t)dim * REC_COLS;           // [MM_STAGE][dim]
    float *ks = qs + (size_t)MM_STAGE * dim;          // [MM_STAGE][dim]
    float *vs = ks + (size_t)MM_STAGE * dim;          // [MM_STAGE][16]
    float *gs = vs + MM_STAGE * REC_COLS;             // [MM_STAGE][2]: log input gate, log forget gate
    float *row = state + (size_t)entry_seat[e] * seat_stride + state_off;
    float *S_g = row + (size_t)h * dim * vdim;
    // (every wavefront reads and writes its own copy of n and m: no wavefront waits for another)
    const int tiles = gridDim.x, tile = blockIdx.x;
    float *n_g = row + (size_t)heads * dim * vdim + ((size_t)h * tiles + tile) * dim;
    float *m_g = row + (size_t)heads * dim * vdim + (size_t)heads * tiles * dim + (size_t)h * tiles + tile;
    for (int r = rg; r < dim; r += REC_ROWGROUPS) {
        S[r * REC_COLS + c] = col_on ? S_g[(size_t)r * vdim + col] : 0.f;
        N[r * REC_COLS + c] = n_g[r];
    }
    float m = *m_g;
    for (int t0 = 0; t0 < n; t0 += MM_STAGE) {
        const int cnt = min(MM_STAGE, n - t0);
        __syncthreads();
        for (int i = lane; i < cnt * dim; i += KVA_WAVE) {
            const int tt = i / dim, r = i % dim;
            const size_t at = (size_t)(q0 + t0 + tt) * y_stride;
            qs[tt * dim + r] = rec_ld(y, y_dtype, at + q_off + h * dim + r) * q_mul;
            ks[tt * dim + r] = rec_ld(y, y_dtype, at + k_off + h * dim + r);
        }
        for (int i = lane; i < cnt * REC_COLS; i += KVA_WAVE) {
            const int tt = i / REC_COLS, cc = i % REC_COLS;
            vs[i] = col0 + cc < vdim ? rec_ld(y, y_dtype, (size_t)(q0 + t0 + tt) * y_stride + v_off + h * vdim + col0 + cc) : 0.f;
        }
        if (lane < cnt) {
            const float zi = gates[(size_t)(q0 + t0 + lane) * 2 * heads + h];
            const float zf = gates[(size_t)(q0 + t0 + lane) * 2 * heads + heads + h];
            const float f = cap * tanhf(zf / cap);
            gs[2 * lane] = cap * tanhf(zi / cap);
            gs[2 * lane + 1] = -rec_softplus(-f);         // logsigmoid
        }
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const float gi = gs[2 * tt], gf = gs[2 * tt + 1];
            const float m_new = fmaxf(gf + m, gi);
            const float keep = expf(gf + m - m_new), take = expf(gi - m_new);
            m = m_new;
            const float tv = take * vs[tt * REC_COLS + c];
            float num = 0.f, nq = 0.f;
            for (int r = rg; r < dim; r += REC_ROWGROUPS) {
                const float kv = ks[tt * dim + r], qv = qs[tt * dim + r];
                const float sv = keep * S[r * REC_COLS + c] + kv * tv;
                const float nv = keep * N[r * REC_COLS + c] + take * kv;
                S[r * REC_COLS + c] = sv;
                N[r * REC_COLS + c] = nv;
                num += sv * qv;
                nq += nv * qv;
            }
            num = rec_column_sum(num);
            nq = rec_column_sum(nq);
            const float den = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
            if (rg == 0 && col_on) out[(size_t)(q0 + t0 + tt) * heads * vdim + (size_t)h * vdim + col] = num / den;
        }
    }
    for (int r = rg; r < dim; r += REC_ROWGROUPS) {
        if (col_on) S_g[(size_t)r * vdim + col] = S[r * REC_COLS + c];
        if (c == 0) n_g[r] = N[r * REC_COLS + c];
    }
    if (lane == 0) *m_g = m;
}

// The same for key sizes up to 128, with the state in registers: a workgroup of four wavefronts takes the 16
// value columns, a wavefront four of them, 16 lanes a column; lane = 16 c + r owns rows r, r + 16, ... of its
// column of S and of its copy of n (RP of each), sums over the rows are rotations inside a row of lanes, and
// the four wavefronts share the staged tokens (32 at a time).
#define MM_REG_STAGE 32
template <int RP>
__global__ void __launch_bounds__(256)
matrix_memory_reg_kernel(float *__restrict__ out, float *__restrict__ state, size_t seat_stride, int state_off,
                         const void *__restrict__ y, int y_dtype, int y_stride, int q_off, int k_off, int v_off,
                         const float *__restrict__ gates, float cap, float q_mul, const int *__restrict__ entry_q_start,
                         const int *__restrict__ entry_seat, int heads, int dim, int vdim) {
    extern __shared__ float lds[];
    const int e = blockIdx.z, h = blockIdx.y, col0 = blockIdx.x * REC_COLS;
    const int q0 = entry_q_start[e], n = entry_q_start[e + 1] - q0;
    if (n <= 0) return;
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE;
    const int r16 = lane % 16, cw = 4 * wave + lane / 16, col = col0 + cw;
    const bool col_on = col < vdim;
    const int dpad = 16 * RP;
    float *qs = lds;                                   // [MM_REG_STAGE][dpad]
    float *ks = qs + MM_REG_STAGE * dpad;              // [MM_REG_STAGE][dpad]
    float *vs = ks + MM_REG_STAGE * dpad;              // [MM_REG_STAGE][16]
    float *gs = vs + MM_REG_STAGE * REC_COLS;          // [MM_REG_STAGE][3]: e^(f + m - m'), e^(i - m'), e^(-m') of every token
    float *row = state + (size_t)entry_seat[e] * seat_stride + state_off;
    float *S_g = row + (size_t)h * dim * vdim;
    const int tiles = gridDim.x, tile = blockIdx.x;
    float *n_g = row + (size_t)heads * dim * vdim + ((size_t)h * tiles + tile) * dim;
    float *m_g = row + (size_t)heads * dim * vdim + (size_t)heads * tiles * dim + (size_t)h * tiles + tile;
    float S[RP], N[RP];
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        const int r = r16 + 16 * i;
        S[i] = (r < dim && col_on) ? S_g[(size_t)r * vdim + col] : 0.f;
        N[i] = r < dim ? n_g[r] : 0.f;
    }
    float m = *m_g;
    // What a thread stages of a chunk of tokens: 2 RP elements of q and of k, 2 of v, and - the first wavefront's
    // lanes - a token's two gate inputs.  All of it is asked for before any of it is used, and the next chunk's
    // while this one's tokens are walked.
    constexpr int PER = MM_REG_STAGE * 16 * RP / 256;
    float pq[PER], pk[PER], pv[2], pzi = 0.f, pzf = 0.f;
    auto fetch = [&](int t0) {
        const int cnt = min(MM_REG_STAGE, n - t0);
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = threadIdx.x + j * 256, tt = i / dpad, r = i % dpad;
            const bool in = tt < cnt && r < dim;
            const size_t at = (size_t)(q0 + t0 + (in ? tt : 0)) * y_stride + h * dim + (in ? r : 0);
            pq[j] = in ? rec_ld(y, y_dtype, at + q_off) * q_mul : 0.f;
            pk[j] = in ? rec_ld(y, y_dtype, at + k_off) : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int i = threadIdx.x + j * 256, tt = i / REC_COLS, cc = i % REC_COLS;
            const bool in = tt < cnt && col0 + cc < vdim;
            pv[j] = in ? rec_ld(y, y_dtype, (size_t)(q0 + t0 + tt) * y_stride + v_off + h * vdim + col0 + cc) : 0.f;
        }
        if (threadIdx.x < cnt) {
            pzi = gates[(size_t)(q0 + t0 + threadIdx.x) * 2 * heads + h];
            pzf = gates[(size_t)(q0 + t0 + threadIdx.x) * 2 * heads + heads + h];
        }
    };
    fetch(0);
    for (int t0 = 0; t0 < n; t0 += MM_REG_STAGE) {
        const int cnt = min(MM_REG_STAGE, n - t0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            qs[threadIdx.x + j * 256] = pq[j];
            ks[threadIdx.x + j * 256] = pk[j];
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) vs[threadIdx.x + j * 256] = pv[j];
        if (wave == 0) {
            // The running maxima of the staged tokens, by the first wavefront, lane = token: with F_t the sum of
            // the log forget gates up to t, m_t = F_t + max(m, max_(j <= t) (i_j - F_j)) - a prefix sum and a
            // prefix maximum over the lanes instead of a walk - and from them what the walk below multiplies by.
            const bool on = lane < cnt;
            float gi = -INFINITY, gf = 0.f;
            if (on) {
                gi = cap * tanhf(pzi / cap);
                gf = -rec_softplus(-cap * tanhf(pzf / cap));
            }
            float F = gf;
#pragma unroll
            for (int o = 1; o < MM_REG_STAGE; o <<= 1) {
                const float up = __shfl_up(F, o, KVA_WAVE);
                if (lane >= o) F += up;
            }
            float A = gi - F;
#pragma unroll
            for (int o = 1; o < MM_REG_STAGE; o <<= 1) {
                const float up = __shfl_up(A, o, KVA_WAVE);
                if (lane >= o) A = fmaxf(A, up);
            }
            const float mt = F + fmaxf(m, A);
            float prev = __shfl_up(mt, 1, KVA_WAVE);
            if (lane == 0) prev = m;
            if (on) {
                gs[3 * lane] = expf(gf + prev - mt);
                gs[3 * lane + 1] = expf(gi - mt);
                gs[3 * lane + 2] = expf(-mt);
            }
            m = __shfl(mt, cnt - 1, KVA_WAVE);
        }
        __syncthreads();
        if (t0 + MM_REG_STAGE < n) fetch(t0 + MM_REG_STAGE);
        for (int tt = 0; tt < cnt; ++tt) {
            const float keep = gs[3 * tt], take = gs[3 * tt + 1], floor_den = gs[3 * tt + 2];
            const float tv = take * vs[tt * REC_COLS + cw];
            float num = 0.f, nq = 0.f;
#pragma unroll
            for (int i = 0; i < RP; ++i) {
                const float kv = ks[tt * dpad + r16 + 16 * i], qv = qs[tt * dpad + r16 + 16 * i];
                S[i] = keep * S[i] + kv * tv;
                N[i] = keep * N[i] + take * kv;
                num += S[i] * qv;
                nq += N[i] * qv;
            }
            num = row16_sum(num);
            nq = row16_sum(nq);
            if (r16 == 0 && col_on)
                out[(size_t)(q0 + t0 + tt) * heads * vdim + (size_t)h * vdim + col] = num / (fmaxf(fabsf(nq), floor_den) + 1e-6f);
        }
    }
#pragma unroll
    for (int i = 0; i < RP; ++i) {
        const int r = r16 + 16 * i;
        if (r < dim && col_on) S_g[(size_t)r * vdim + col] = S[i];
        if (r < dim && cw == 0) n_g[r] = N[i];
    }
    if (threadIdx.x == 0) *m_g = m;
}

extern "C" int kva_matrix_memory_state(int heads, int dim, int vdim) {
    const int tiles = (vdim + REC_COLS - 1) / REC_COLS;
    return heads * dim * vdim + heads * tiles * (dim + 1);
}

extern "C" int kva_matrix_memory(float *out, float *state, long long seat_stride, int state_off, const void *y, int y_dtype,
                                 int y_stride, int q_off, int k_off, int v_off, const float *gates, float cap, float q_mul,
                                 const int *entry_q_start, const int *entry_seat, int entries, int heads, int dim, int vdim,
                                 hipStream_t stream) {
    KVA_REQUIRE(out && state && y && gates && entry_q_start && entry_seat, "matrix_memory: missing operand");
    KVA_REQUIRE(heads > 0 && dim > 0 && dim <= REC_MAX_DIM && vdim > 0 && cap > 0.f, "matrix_memory: bad sizes (key size up to %d)", REC_MAX_DIM);
    KVA_REQUIRE(entries >= 0 && entries <= 65535 && heads <= 65535, "matrix_memory: bad batch");
    if (entries == 0) return KVA_OK;
    const dim3 grid((vdim + REC_COLS - 1) / REC_COLS, heads, entries);
    if (dim <= 128) {
        // (which kernel runs depends on the key size alone: a token's numbers are the same in any batch)
        const int rp = dim <= 16 ? 1 : dim <= 32 ? 2 : dim <= 64 ? 4 : 8;
        const size_t reg_lds = ((size_t)2 * MM_REG_STAGE * 16 * rp + MM_REG_STAGE * REC_COLS + 3 * MM_REG_STAGE) * sizeof(float);
#define KVA_MM_REG(RP)                                                                                                      \
    hipLaunchKernelGGL(matrix_memory_reg_kernel<RP>, grid, dim3(256), reg_lds, stream, out, state, (size_t)seat_stride,     \
                       state_off, y, y_dtype, y_stride, q_off, k_off, v_off, gates, cap, q_mul, entry_q_start, entry_seat,  \
                       heads, dim, vdim)
        if (rp == 1) KVA_MM_REG(1);
        else if (rp == 2) KVA_MM_REG(2);
        else if (rp == 4) KVA_MM_REG(4);
        else KVA_MM_REG(8);
#undef KVA_MM_REG
        KVA_CHECK_LAUNCH("matrix_memory");
        return KVA_OK;
    }
    const size_t lds = ((size_t)2 * dim * REC_COLS + (size_t)2 * MM_STAGE * dim + MM_STAGE * REC_COLS + 2 * MM_STAGE) * sizeof(float);
    KVA_REQUIRE(lds <= 160 * 1024, "matrix_memory: a key size of %d does not fit the local memory", dim);
    if (lds > 64 * 1024)
        hipFuncSetAttribute(reinterpret_cast<const void *>(matrix_memory_kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(matrix_memory_kernel, dim3((vdim + REC_COLS - 1) / REC_COLS, heads, entries), dim3(KVA_WAVE), lds, stream,
                       out, state, (size_t)seat_stride, state_off, y, y_dtype, y_stride, q_off, k_off, v_off, gates, cap, q_mul,
                       entry_q_start, entry_seat, heads, dim, vdim);
    KVA_CHECK_LAUNCH("matrix_memory");
    return KVA_OK;
}
