// Position encoding of queries and keys with the cache write, for the variants that the
// rotate-half kernel (rope_cache.hip) does not cover:
//
//  * kva_qk_encode_cache: heads of queries and keys whose first `rot` elements are rotated with
//    either pairing (pair i = elements (i, i + rot/2) or (2i, 2i + 1)), optionally followed by a
//    division of every head by its root mean square (and a multiplication by a weight per element,
//    one for queries and one for keys: an RMS norm of every head) - or, with norm_first, preceded by it; keys of `head_dim` and values of another
//    size `value_dim` go to the paged K / V^T arrays (kv_layout.h).
//  * kva_latent_encode_cache: a low-rank key/value entry.  Per token one latent vector of `rank`
//    elements, RMS-normed with a weight, and one rotated key part of `rot` elements shared by all
//    heads are stored side by side in a row of `rank + rot`; the rotated part of every query head
//    is written behind that head's `rank` columns of the query buffer the attention kernel reads.
//
// cos and sin come from fp32 tables [positions, rot / 2]; all arithmetic is fp32.
#include "common.h"
#include "kv_layout.h"
#include <math.h>

#define ENC_MAX_HEAD_DIM 512

template <typename T>
__global__ void __launch_bounds__(256)
qk_encode_cache_kernel(T *__restrict__ qkv, int row_stride, int k_off, int v_off, T *__restrict__ k_cache,
                       T *__restrict__ v_cache, const float *__restrict__ cos_table,
                       const float *__restrict__ sin_table, const int *__restrict__ positions,
                       const int *__restrict__ slot_mapping, int num_q_heads, int num_kv_heads, int head_dim,
                       int value_dim, int rot, int interleaved, float unit_eps, int page_size,
                       const T *__restrict__ bias, const float *__restrict__ q_weight,
                       const float *__restrict__ k_weight, int norm_first) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE, waves = blockDim.x / KVA_WAVE;
    T *row = qkv + (size_t)t * row_stride;
    const int pos = positions[t];
    const int half = rot / 2, pairs = head_dim / 2;
    const float *cs = cos_table + (size_t)pos * half, *sn = sin_table + (size_t)pos * half;
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
    constexpr int PER = ENC_MAX_HEAD_DIM / 2 / KVA_WAVE;

    for (int head = wave; head < num_q_heads + num_kv_heads; head += waves) {
        const bool is_q = head < num_q_heads;
        if (!is_q && slot < 0) continue;
        T *h = is_q ? row + (size_t)head * head_dim : row + k_off + (size_t)(head - num_q_heads) * head_dim;
        // (optional) the projection's bias, laid out [q heads | k heads | v heads] without gaps
        const T *hb = bias ? bias + (size_t)head * head_dim : nullptr;
        float o1[PER], o2[PER];
        int i1[PER], i2[PER];
        float sq = 0.f;
#pragma unroll
        for (int c = 0; c < PER; ++c) {
            const int p = lane + c * KVA_WAVE;
            o1[c] = o2[c] = 0.f;
            i1[c] = i2[c] = 0;
            if (p >= pairs) continue;
            // pair p of the head: a rotated pair while p < rot / 2, two plain neighbours behind
            if (interleaved) {
                i1[c] = 2 * p;
                i2[c] = 2 * p + 1;
            } else if (p < half) {
                i1[c] = p;
                i2[c] = p + half;
            } else {
                i1[c] = rot + 2 * (p - half);
                i2[c] = i1[c] + 1;
            }
            const float u = to_float(h[i1[c]]) + (hb ? to_float(hb[i1[c]]) : 0.f);
            const float v = to_float(h[i2[c]]) + (hb ? to_float(hb[i2[c]]) : 0.f);
            if (p < half && !norm_first) {
                const float co = cs[p], si = sn[p];
                o1[c] = u * co - v * si;
                o2[c] = v * co + u * si;
            } else {
                o1[c] = u;
                o2[c] = v;
            }
            sq += o1[c] * o1[c] + o2[c] * o2[c];
        }
        float mul = 1.f;
        if (unit_eps >= 0.f) mul = 1.0f / sqrtf(wave_sum(sq) / (float)head_dim + unit_eps);
        // (optional) the weight of an RMS norm over the head, one per element, shared by the heads
        const float *nw = is_q ? q_weight : k_weight;
        T *kdst = nullptr;
        const int kc = kva_k_chunk(head_dim);
        if (!is_q) kdst = k_cache + ((size_t)page * num_kv_heads + (head - num_q_heads)) * page_size * head_dim;
#pragma unroll
        for (int c = 0; c < PER; ++c) {
            const int p = lane + c * KVA_WAVE;
            if (p >= pairs) continue;
            float f1 = o1[c] * mul * (nw ? nw[i1[c]] : 1.f), f2 = o2[c] * mul * (nw ? nw[i2[c]] : 1.f);
            if (norm_first && p < half) {           // the normed head is what is rotated
                const float co = cs[p], si = sn[p], u = f1, v = f2;
                f1 = u * co - v * si;
                f2 = v * co + u * si;
            }
            const T r1 = from_float<T>(f1), r2 = from_float<T>(f2);
            if (is_q) {
                h[i1[c]] = r1;
                h[i2[c]] = r2;
            } else {
                kdst[kva_k_at(off, i1[c], page_size, kc)] = r1;
                kdst[kva_k_at(off, i2[c], page_size, kc)] = r2;
            }
        }
    }
    if (slot >= 0) {
        const T *v = row + v_off;
        const T *vb = bias ? bias + (size_t)(num_q_heads + num_kv_heads) * head_dim : nullptr;
        for (int w = threadIdx.x; w < num_kv_heads * value_dim; w += blockDim.x) {
            const int kvh = w / value_dim, j = w % value_dim;
            v_cache[(((size_t)page * num_kv_heads + kvh) * value_dim + j) * page_size + off] =
                vb ? from_float<T>(to_float(v[w]) + to_float(vb[w])) : v[w];
        }
    }
}

// bf16, interleaved pairs, heads of 8 * 2^k elements (up to 512): a lane takes 8 neighbouring
// elements of a head (four whole pairs: 16 bytes in, 16 bytes out - one chunk of the K page), the
// 2^k lanes of a head add their squares up between them.
__global__ void __launch_bounds__(256)
qk_encode_cache_vec_kernel(bf16_t *__restrict__ qkv, int row_stride, int k_off, int v_off, bf16_t *__restrict__ k_cache,
                           bf16_t *__restrict__ v_cache, const float *__restrict__ cos_table,
                           const float *__restrict__ sin_table, const int *__restrict__ positions,
                           const int *__restrict__ slot_mapping, int num_q_heads, int num_kv_heads, int head_dim,
                           int value_dim, int rot, float unit_eps, int page_size) {
    const int t = blockIdx.x;
    bf16_t *row = qkv + (size_t)t * row_stride;
    const int pos = positions[t];
    const int half = rot / 2, vecs = head_dim / 8;                // lanes a head
    const float *cs = cos_table + (size_t)pos * half, *sn = sin_table + (size_t)pos * half;
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
    const int total = (num_q_heads + num_kv_heads) * vecs;
    for (int w0 = 0; w0 < total; w0 += blockDim.x) {              // (uniform trip count: the lanes of a head shuffle)
        const int w = w0 + threadIdx.x;
        const bool on = w < total;
        const int head = on ? w / vecs : 0, j = on ? w % vecs : 0;
        const bool is_q = head < num_q_heads;
        bf16_t *h = is_q ? row + (size_t)head * head_dim : row + k_off + (size_t)(head - num_q_heads) * head_dim;
        float x[8], y[8];
        const uint4 in = *reinterpret_cast<const uint4 *>(h + 8 * j);
        const uint32_t iw[4] = {in.x, in.y, in.z, in.w};
        float sq = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            x[2 * i] = bf16_bits_to_float((uint16_t)(iw[i] & 0xffffu));
            x[2 * i + 1] = bf16_bits_to_float((uint16_t)(iw[i] >> 16));
            const int p = 4 * j + i;                              // pair (2p, 2p + 1) of the head
            if (p < half) {
                const float co = cs[p], si = sn[p];
                y[2 * i] = x[2 * i] * co - x[2 * i + 1] * si;
                y[2 * i + 1] = x[2 * i + 1] * co + x[2 * i] * si;
            } else {
                y[2 * i] = x[2 * i];
                y[2 * i + 1] = x[2 * i + 1];
            }
            sq += y[2 * i] * y[2 * i] + y[2 * i + 1] * y[2 * i + 1];
        }
        float mul = 1.f;
        if (unit_eps >= 0.f) {
            for (int o = vecs / 2; o > 0; o >>= 1) sq += __shfl_xor(sq, o, KVA_WAVE);
            mul = 1.0f / sqrtf(sq / (float)head_dim + unit_eps);
        }
        uint32_t ow[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            ow[i] = (uint32_t)float_to_bf16_bits(y[2 * i] * mul) | ((uint32_t)float_to_bf16_bits(y[2 * i + 1] * mul) << 16);
        const uint4 res = make_uint4(ow[0], ow[1], ow[2], ow[3]);
        if (!on) continue;
        if (is_q) {
            *reinterpret_cast<uint4 *>(h + 8 * j) = res;
        } else if (slot >= 0) {
            bf16_t *kdst = k_cache + ((size_t)page * num_kv_heads + (head - num_q_heads)) * page_size * head_dim;
            *reinterpret_cast<uint4 *>(kdst + kva_k_at(off, 8 * j, page_size, 8)) = res;
        }
    }
    if (slot >= 0) {
        const bf16_t *v = row + v_off;
        for (int w = threadIdx.x; w < num_kv_heads * value_dim; w += blockDim.x) {
            const int kvh = w / value_dim, j = w % value_dim;
            v_cache[(((size_t)page * num_kv_heads + kvh) * value_dim + j) * page_size + off] = v[w];
        }
    }
}

extern "C" int kva_qk_encode_cache(void *qkv, int row_stride, int k_off, int v_off, void *k_cache, void *v_cache,
                                   const float *cos_table, const float *sin_table, const int *positions,
                                   const int *slot_mapping, int tokens, int num_q_heads, int num_kv_heads,
                                   int head_dim, int value_dim, int rot, int interleaved, float unit_eps,
                                   int page_size, int dtype, const void *bias, const float *q_weight,
                                   const float *k_weight, int norm_first, hipStream_t stream) {
    // norm_first: the division by the root mean square (and the weight) comes before the rotation
    KVA_REQUIRE(!norm_first || unit_eps >= 0.f, "qk_encode_cache: a norm before the rotation needs the norm");
    // (num_kv_heads = 0: rows of queries alone, for a layer that reads another layer's keys and values)
    KVA_REQUIRE(tokens >= 0 && num_q_heads > 0 && num_kv_heads >= 0 && value_dim > 0, "qk_encode_cache: bad sizes");
    KVA_REQUIRE(num_kv_heads > 0 || !slot_mapping, "qk_encode_cache: a cache write without key heads");
    KVA_REQUIRE((!q_weight && !k_weight) || unit_eps >= 0.f, "qk_encode_cache: a norm weight without the norm");
    KVA_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= ENC_MAX_HEAD_DIM,
                "qk_encode_cache: head_dim %d must be even and at most %d", head_dim, ENC_MAX_HEAD_DIM);
    KVA_REQUIRE(rot >= 0 && rot <= head_dim && rot % 2 == 0,
                "qk_encode_cache: %d rotated elements must be even and at most head_dim %d", rot, head_dim);
    KVA_REQUIRE(rot == 0 || (cos_table && sin_table), "qk_encode_cache: a rotation needs both tables");
    KVA_REQUIRE(!slot_mapping || (k_cache && v_cache && page_size > 0),
                "qk_encode_cache: cache write asked for without cache or page size");
    KVA_REQUIRE(k_off >= num_q_heads * head_dim && v_off >= k_off + num_kv_heads * head_dim &&
                    row_stride >= v_off + num_kv_heads * value_dim,
                "qk_encode_cache: the row layout [q | k | v] does not fit its stride");
    if (tokens == 0) return KVA_OK;
    if (rot == 0) cos_table = sin_table = reinterpret_cast<const float *>(qkv);     // never read
    const int vecs = head_dim / 8;
    if (!bias && !q_weight && !k_weight && !norm_first && dtype == KVA_BF16 && interleaved && head_dim % 8 == 0 && (vecs & (vecs - 1)) == 0 && vecs <= KVA_WAVE &&
        row_stride % 8 == 0 && k_off % 8 == 0 && (reinterpret_cast<uintptr_t>(qkv) & 15) == 0) {
        hipLaunchKernelGGL(qk_encode_cache_vec_kernel, dim3(tokens), dim3(256), 0, stream, (bf16_t *)qkv, row_stride,
                           k_off, v_off, (bf16_t *)k_cache, (bf16_t *)v_cache, cos_table, sin_table, positions,
                           slot_mapping, num_q_heads, num_kv_heads, head_dim, value_dim, rot, unit_eps, page_size);
        KVA_CHECK_LAUNCH("qk_encode_cache");
        return KVA_OK;
    }
    if (dtype == KVA_F32)
        hipLaunchKernelGGL(qk_encode_cache_kernel<float>, dim3(tokens), dim3(256), 0, stream, (float *)qkv, row_stride,
                           k_off, v_off, (float *)k_cache, (float *)v_cache, cos_table, sin_table, positions,
                           slot_mapping, num_q_heads, num_kv_heads, head_dim, value_dim, rot, interleaved, unit_eps,
                           page_size, (const float *)bias, q_weight, k_weight, norm_first);
    else if (dtype == KVA_BF16)
        hipLaunchKernelGGL(qk_encode_cache_kernel<bf16_t>, dim3(tokens), dim3(256), 0, stream, (bf16_t *)qkv,
                           row_stride, k_off, v_off, (bf16_t *)k_cache, (bf16_t *)v_cache, cos_table, sin_table,
                           positions, slot_mapping, num_q_heads, num_kv_heads, head_dim, value_dim, rot, interleaved,
                           unit_eps, page_size, (const bf16_t *)bias, q_weight, k_weight, norm_first);
    else KVA_REQUIRE(false, "qk_encode_cache: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("qk_encode_cache");
    return KVA_OK;
}

// rotates pair i of `rot` elements at src into dst (which may be src); cs / sn: this position's row
template <typename T>
__device__ inline void rotate_pair(const T *src, T *dst, int i, int rot, int interleaved, const float *cs,
                                   const float *sn) {
    const int a = interleaved ? 2 * i : i, b = interleaved ? 2 * i + 1 : i + rot / 2;
    const float u = to_float(src[a]), v = to_float(src[b]);
    const float co = cs[i], si = sn[i];
    dst[a] = from_float<T>(u * co - v * si);
    dst[b] = from_float<T>(v * co + u * si);
}

// y row: [H heads of (plain_dim + rot) | ... ] with the compressed entry (rank + rot) at kv_off.
template <typename T, typename TW>
__global__ void __launch_bounds__(256)
latent_encode_cache_kernel(const T *__restrict__ y, int row_stride, int kv_off, T *__restrict__ q_lat,
                           T *__restrict__ cache, T *__restrict__ cache_t, int page_size,
                           const TW *__restrict__ norm_weight, float eps,
                           const float *__restrict__ cos_table, const float *__restrict__ sin_table,
                           const int *__restrict__ positions, const int *__restrict__ slot_mapping, int heads,
                           int plain_dim, int rank, int rot, int interleaved) {
    __shared__ float red_s[4];
    const int t = blockIdx.x;
    const T *row = y + (size_t)t * row_stride;
    const int pos = positions[t], half = rot / 2, kd = rank + rot;
    const float *cs = cos_table + (size_t)pos * half, *sn = sin_table + (size_t)pos * half;
    // the rotated part of every query head, behind the head's `rank` absorbed columns
    for (int w = threadIdx.x; w < heads * half; w += blockDim.x) {
        const int h = w / half, i = w % half;
        rotate_pair(row + (size_t)h * (plain_dim + rot) + plain_dim, q_lat + ((size_t)t * heads + h) * kd + rank, i, rot,
                    interleaved, cs, sn);
    }
    const int slot = slot_mapping ? slot_mapping[t] : -1;       // uniform over the workgroup
    if (slot < 0) return;
    const T *c = row + kv_off;
    T *dst = cache + (size_t)slot * kd;
    float sq = 0.f;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) {
        const float v = to_float(c[j]);
        sq += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, red_s, blockDim.x / KVA_WAVE) / (float)rank + eps);
    // (the latent a second time, transposed inside its page [rank, page_size], where a kernel reads it that way)
    T *dst_t = cache_t ? cache_t + (size_t)(slot / page_size) * rank * page_size + slot % page_size : nullptr;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) {
        const T v = from_float<T>(to_float(c[j]) * inv * to_float(norm_weight[j]));
        dst[j] = v;
        if (dst_t) dst_t[(size_t)j * page_size] = v;
    }
    for (int i = threadIdx.x; i < half; i += blockDim.x) rotate_pair(c + rank, dst + rank, i, rot, interleaved, cs, sn);
}

extern "C" int kva_latent_encode_cache(const void *y, int row_stride, int kv_off, void *q_lat, void *cache,
                                       void *cache_t, int page_size, const void *norm_weight, int weight_dtype, float eps, const float *cos_table,
                                       const float *sin_table, const int *positions, const int *slot_mapping,
                                       int tokens, int heads, int plain_dim, int rank, int rot, int interleaved,
                                       int dtype, hipStream_t stream) {
    KVA_REQUIRE(tokens >= 0 && heads > 0 && plain_dim > 0 && rank > 0, "latent_encode_cache: bad sizes");
    KVA_REQUIRE(rot > 0 && rot % 2 == 0 && cos_table && sin_table,
                "latent_encode_cache: %d rotated elements must be even and positive, with both tables", rot);
    KVA_REQUIRE(kv_off >= heads * (plain_dim + rot) && row_stride >= kv_off + rank + rot,
                "latent_encode_cache: the row layout [queries | entry] does not fit its stride");
    KVA_REQUIRE(!slot_mapping || cache, "latent_encode_cache: cache write asked for without a cache");
    KVA_REQUIRE(!cache_t || page_size > 0, "latent_encode_cache: the transposed copy needs the page size");
    KVA_REQUIRE(dtype == KVA_F32 || dtype == KVA_BF16, "latent_encode_cache: unsupported dtype %d", dtype);
    if (tokens == 0) return KVA_OK;
#define LAUNCH_LE(T, TW)                                                                                        \
    hipLaunchKernelGGL((latent_encode_cache_kernel<T, TW>), dim3(tokens), dim3(256), 0, stream, (const T *)y,   \
                       row_stride, kv_off, (T *)q_lat, (T *)cache, (T *)cache_t, page_size,                     \
                       (const TW *)norm_weight, eps, cos_table,                                                 \
                       sin_table, positions, slot_mapping, heads, plain_dim, rank, rot, interleaved)
    if (dtype == KVA_F32 && weight_dtype == KVA_F32) LAUNCH_LE(float, float);
    else if (dtype == KVA_BF16 && weight_dtype == KVA_BF16) LAUNCH_LE(bf16_t, bf16_t);
    else if (dtype == KVA_BF16 && weight_dtype == KVA_F32) LAUNCH_LE(bf16_t, float);
    else KVA_REQUIRE(false, "latent_encode_cache: a 32-bit entry needs a 32-bit norm weight");
#undef LAUNCH_LE
    KVA_CHECK_LAUNCH("latent_encode_cache");
    return KVA_OK;
}
