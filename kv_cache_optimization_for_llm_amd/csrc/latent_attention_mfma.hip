// Attention over low-rank entries on the matrix cores (bf16, gfx950): prompt portions and decoded
// tokens, one kernel.
//
// Every token keeps one row [latent (RANK) ; rotated key part] of KD elements for all heads
// (parts/latent_attention.py), in pages [page_size, KD], and the latent a second time transposed,
// pages [RANK, page_size].  A head's query is a row of the same KD elements, so all H heads of a
// token attend over the same rows: the 16 rows of a matrix-core tile are (token, head) pairs,
// row = token_in_entry * H + head, and each row a wavefront loads serves up to 16 heads.
//
// As in attention_mfma.hip everything is computed transposed so that both operands come from
// memory in operand layout, without LDS:
//     S^T = K  Q^T   A = 16 rows of the cache x 32 of their elements (16 bytes a lane, row-major)
//     O^T = C^T P^T  A = 16 latent elements x 32 keys, from the transposed copy; the matrix core's
//                    k index of this product is the permutation of the 32 keys in which S^T left
//                    P in the registers (lane group g, element j <-> key (j / 4) * 16 + 4 g + j % 4)
// Softmax is online in fp32, base 2.  A work item is (16 rows of one entry, a range of keys); an
// item writes the normalised bf16 result itself when its range is all keys, otherwise an
// un-normalised partial (o, m, l) that latent_merge_kernel combines.  The sink of a head (one more
// term exp(sink) of its denominator) is added where the result is normalised.
#include "common.h"
#include "attention_frag.h"
#include "kv_layout.h"
#include <math.h>

#define LAT_LOG2E 1.44269504088896340736f

// The body; two kernels below give it one or up to four wavefronts a SIMD.  A block's loads are
// all asked for before its first product (a load inside the product loop compiles to one trip to
// memory per product): the 2 NKS key fragments at once, the value fragments eight tiles ahead.
// The queries wait in LDS (one wavefront's 16 rows), so that the registers hold the keys in flight.
template <int NDT /* RANK / 16 */, int NKS /* KD / 32 */>
__device__ __forceinline__ void
latent_attention_mfma_body(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                             const bf16_t *__restrict__ q, const bf16_t *__restrict__ cache,
                             const bf16_t *__restrict__ cache_t, const int *__restrict__ block_table, int max_blocks,
                             const int *__restrict__ item_entry, const int *__restrict__ item_row0,
                             const int *__restrict__ entry_seat, const int *__restrict__ entry_q_start,
                             const int *__restrict__ entry_start_pos, int heads, int page_size, float scale,
                             int window, int keep_first, const float *__restrict__ sinks, int splits, int per_split) {
    constexpr int RANK = NDT * 16, KD = NKS * 32;
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int item = blockIdx.x, split = blockIdx.y;
    const int e = item_entry[item], row0 = item_row0[item];
    const int q_start = entry_q_start[e], q_len = entry_q_start[e + 1] - q_start;
    const int start_pos = entry_start_pos[e];
    const int *bt = block_table + (size_t)entry_seat[e] * max_blocks;
    const int rows = q_len * heads;                         // rows of the entry
    const int last_row = min(row0 + 15, rows - 1);
    const int item_hi = start_pos + last_row / heads;       // newest key any row of the item sees
    const int pos_lo = start_pos + row0 / heads;            // position of the item's first row
    const int my_row = min(row0 + r, rows - 1);
    const bool row_valid = row0 + r < rows;
    const int my_pos = start_pos + my_row / heads;
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int item_lo = (window > 0 && pos_lo - window + 1 > 0) ? pos_lo - window + 1 : 0;
    const int hi_lo = (window > 0 && item_hi - window + 1 > 0) ? item_hi - window + 1 : 0;     // where the last row's window starts
    const size_t my_global = (size_t)q_start * heads + my_row;      // row of q / out

    // Q^T in operand layout: lane (row r, group g) holds elements 32 ks + 8 g .. + 7 of its row;
    // kept in LDS as [ks][lane] (a lane reads back what it wrote: no barrier)
    __shared__ uint4 q_s[NKS * KVA_WAVE];
    {
        const bf16_t *qrow = q + my_global * KD + 8 * g;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) q_s[ks * KVA_WAVE + lane] = *reinterpret_cast<const uint4 *>(qrow + 32 * ks);
    }
    f32x4 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;                           // m in the base-2 domain, l this lane's part
    const float scale2 = scale * LAT_LOG2E;

    int k_begin = 0, k_end = item_hi + 1;
    if (splits > 1) {
        k_begin = split * per_split;
        k_end = min(k_end, k_begin + per_split);
    }
    for (int kstart = k_begin & ~31; kstart < k_end; kstart += 32) {
        // nothing of the block is visible: behind every row's window and past the kept positions
        if (kstart + 32 <= item_lo && kstart >= keep_first) continue;
        // the two 16-key tiles of the block lie in one page each (pages hold a multiple of 16 keys)
        int page[2];
        bool mapped[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key0 = kstart + 16 * t;
            const int p = key0 <= item_hi ? bt[key0 / page_size] : -1;
            mapped[t] = p >= 0;
            page[t] = p >= 0 ? p : 0;                       // a tile nobody sees is read from a page that exists
        }
        f32x4 s[2];
        Frag8 kf[2][NKS];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key = kstart + 16 * t + r;
            const bf16_t *krow = cache + ((size_t)page[t] * page_size + key % page_size) * KD + 8 * g;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) kf[t][ks].u4 = *reinterpret_cast<const uint4 *>(krow + 32 * ks);
        }
        __builtin_amdgcn_sched_barrier(0);              // every key load of the block is out before the first product
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                Frag8 qf;
                qf.u4 = q_s[ks * KVA_WAVE + lane];
                s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][ks].v, qf.v, s[t], 0, 0, 0);
            }
        }
        // mask and online softmax: lane (row r, group g) holds keys kstart + 16 t + 4 g + i
        // a block that every row of the item sees whole (the common one) needs no mask: wave-uniform
        const bool whole = mapped[0] && mapped[1] && kstart >= k_begin && kstart + 32 <= k_end && kstart + 31 <= pos_lo &&
                           (kstart >= hi_lo || kstart + 32 <= keep_first);
        float sv[8], mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float x = s[t][i] * scale2;
                if (!whole) {
                    const int key = kstart + 16 * t + 4 * g + i;
                    const bool vis = row_valid && mapped[t] && key <= my_pos && (key >= my_lo || key < keep_first) &&
                                     key >= k_begin && key < k_end;
                    x = vis ? x : -INFINITY;
                }
                sv[t * 4 + i] = x;
                mx = fmaxf(mx, x);
            }
        // the running maximum moves in few blocks: only then are l and O re-based (wave-uniform branch)
        const float bm = quad_rows_max(mx);
        if (__builtin_amdgcn_ballot_w64(bm > m) != 0) {
            const float m_new = fmaxf(m, bm);
            const float corr = __builtin_amdgcn_exp2f(m - ((m_new == -INFINITY) ? 0.f : m_new));     // exp2(-inf) = 0
            l *= corr;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) {
                o[dt][0] *= corr; o[dt][1] *= corr; o[dt][2] *= corr; o[dt][3] *= corr;
            }
            m = m_new;
        }
        const float ref = (m == -INFINITY) ? 0.f : m;
        Frag8 pf;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            const float p0 = __builtin_amdgcn_exp2f(sv[j] - ref), p1 = __builtin_amdgcn_exp2f(sv[j + 1] - ref);
            l += p0 + p1;
            pf.p2[j / 2] = pack_bf16(p0, p1);
        }
        // O^T += C^T P^T.  Lane (latent element r of the tile, group g) takes keys 4 g .. 4 g + 3 of
        // each 16-key tile: 8 bytes of the transposed page.  Keys that no row of this item may see
        // (past its newest, outside this range, an unmapped tile) are made zero: their
        // probabilities are, and zero times whatever a page held before must stay zero.
        uint2 keep[2];
        const bf16_t *vrow[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key0 = kstart + 16 * t + 4 * g;
            int n = min(item_hi + 1, k_end) - key0;                   // leading keys of the four that count
            if (!mapped[t] || key0 + 4 <= k_begin) n = 0;
            keep[t] = keep_first_keys(make_uint2(~0u, ~0u), n);
            if (key0 < k_begin && n > 0) {                             // a range that starts inside the four
                const uint2 head = keep_first_keys(make_uint2(~0u, ~0u), k_begin - key0);
                keep[t].x &= ~head.x; keep[t].y &= ~head.y;
            }
            vrow[t] = cache_t + ((size_t)page[t] * RANK + r) * page_size + key0 % page_size;
        }
        constexpr int VC = NDT < 8 ? NDT : 8;                          // value tiles asked for together
#pragma unroll
        for (int d0 = 0; d0 < NDT; d0 += VC) {
            Frag8 vv[VC];
#pragma unroll
            for (int j = 0; j < VC; ++j) {
                vv[j].u2[0] = *reinterpret_cast<const uint2 *>(vrow[0] + (size_t)(d0 + j) * 16 * page_size);
                vv[j].u2[1] = *reinterpret_cast<const uint2 *>(vrow[1] + (size_t)(d0 + j) * 16 * page_size);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < VC; ++j) {
                vv[j].u2[0].x &= keep[0].x; vv[j].u2[0].y &= keep[0].y;
                vv[j].u2[1].x &= keep[1].x; vv[j].u2[1].y &= keep[1].y;
                o[d0 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv[j].v, pf.v, o[d0 + j], 0, 0, 0);
            }
        }
    }
    l = quad_rows_sum(l);
    if (!row_valid) return;
    // lane (row r, group g) holds O^T[16 dt + 4 g + i][row r]
    if (splits > 1) {
        float *po = part_o + (my_global * splits + split) * RANK + 4 * g;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<float4 *>(po + 16 * dt) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
        if (g == 0) {
            part_ml[(my_global * splits + split) * 2] = m;
            part_ml[(my_global * splits + split) * 2 + 1] = l;
        }
        return;
    }
    float mul = 1.f;
    if (sinks) {
        const float sk = sinks[my_row % heads] * LAT_LOG2E, m_new = fmaxf(m, sk);
        const float corr = __builtin_amdgcn_exp2f(m - m_new);
        l = l * corr + __builtin_amdgcn_exp2f(sk - m_new);
        mul = corr;
    }
    mul /= l;
    bf16_t *orow = out + my_global * RANK + 4 * g;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
        Frag4 w;
        w.h[0] = float_to_bf16_bits(o[dt][0] * mul); w.h[1] = float_to_bf16_bits(o[dt][1] * mul);
        w.h[2] = float_to_bf16_bits(o[dt][2] * mul); w.h[3] = float_to_bf16_bits(o[dt][3] * mul);
        *reinterpret_cast<uint2 *>(orow + 16 * dt) = w.u2;
    }
}

#define LAT_KERNEL_ARGS                                                                                        \
    bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml, const bf16_t *__restrict__ q, \
        const bf16_t *__restrict__ cache, const bf16_t *__restrict__ cache_t, const int *__restrict__ block_table, \
        int max_blocks, const int *__restrict__ item_entry, const int *__restrict__ item_row0,                \
        const int *__restrict__ entry_seat, const int *__restrict__ entry_q_start,                            \
        const int *__restrict__ entry_start_pos, int heads, int page_size, float scale, int window,           \
        int keep_first, const float *__restrict__ sinks, int splits, int per_split
#define LAT_KERNEL_PASS                                                                                        \
    out, part_o, part_ml, q, cache, cache_t, block_table, max_blocks, item_entry, item_row0, entry_seat,       \
        entry_q_start, entry_start_pos, heads, page_size, scale, window, keep_first, sinks, splits, per_split

template <int NDT, int NKS>
__global__ void __launch_bounds__(KVA_WAVE) latent_attention_mfma_kernel(LAT_KERNEL_ARGS) {
    latent_attention_mfma_body<NDT, NKS>(LAT_KERNEL_PASS);
}

// large rows: one wavefront a SIMD, so that a block's keys (2 NKS fragments) fit the registers beside the result
template <int NDT, int NKS>
__global__ void __launch_bounds__(KVA_WAVE) __attribute__((amdgpu_waves_per_eu(1, 1)))
latent_attention_mfma_wide_kernel(LAT_KERNEL_ARGS) {
    latent_attention_mfma_body<NDT, NKS>(LAT_KERNEL_PASS);
}

// out[row] = sum_s w_s o_s / (sum_s w_s l_s + exp(sink)), w_s = exp2(m_s - max); one workgroup a row
__global__ void __launch_bounds__(256)
latent_merge_kernel(bf16_t *__restrict__ out, const float *__restrict__ part_o, const float *__restrict__ part_ml,
                    const float *__restrict__ sinks, int heads, int rank, int splits) {
    const size_t row = blockIdx.x;
    const float *ml = part_ml + row * splits * 2;
    float m = sinks ? sinks[row % heads] * LAT_LOG2E : -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, ml[2 * s]);
    float den = sinks ? __builtin_amdgcn_exp2f(sinks[row % heads] * LAT_LOG2E - m) : 0.f;
    for (int s = 0; s < splits; ++s) den += __builtin_amdgcn_exp2f(ml[2 * s] - m) * ml[2 * s + 1];
    // (a range without a visible key - most of them under a window or chunks - has l = 0 and is not read;
    // the order of the others stays, so the sum does not depend on how many empty ones lie between)
    for (int j = threadIdx.x; j < rank; j += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s)
            if (ml[2 * s + 1] != 0.f)
                acc += __builtin_amdgcn_exp2f(ml[2 * s] - m) * part_o[(row * splits + s) * rank + j];
        out[row * rank + j].bits = float_to_bf16_bits(acc / den);
    }
}

// The (rank, row size) pairs with an instance.
#define LAT_INSTANCES(X) X(4, 3) X(4, 4) X(8, 5) X(8, 6) X(16, 9) X(16, 10) X(32, 18) X(24, 14)

extern "C" int kva_latent_attention_mfma_supported(int rank, int key_dim, int page_size) {
    if (page_size <= 0 || page_size % 16) return 0;
#define CHECK_ONE(NDT, NKS) if (rank == NDT * 16 && key_dim == NKS * 32) return 1;
    LAT_INSTANCES(CHECK_ONE)
#undef CHECK_ONE
    return 0;
}

extern "C" int kva_latent_attention_mfma(void *out, float *part_o, float *part_ml, const void *q, const void *cache,
                                         const void *cache_t, const int *block_table, int max_blocks,
                                         const int *item_entry, const int *item_row0, const int *entry_seat,
                                         const int *entry_q_start, const int *entry_start_pos, int num_items,
                                         int total_rows, int heads, int rank, int key_dim, int page_size, float scale,
                                         int window, int keep_first, const float *sinks, int splits, int per_split,
                                         hipStream_t stream) {
    KVA_REQUIRE(kva_latent_attention_mfma_supported(rank, key_dim, page_size),
                "latent_attention_mfma: no instance for rank %d, rows of %d, pages of %d", rank, key_dim, page_size);
    KVA_REQUIRE(num_items >= 0 && heads > 0 && max_blocks > 0 && total_rows >= 0, "latent_attention_mfma: bad sizes");
    KVA_REQUIRE(splits >= 1 && splits <= 65535 && (splits == 1 || (per_split > 0 && per_split % 32 == 0 && part_o && part_ml)),
                "latent_attention_mfma: key ranges need a length that is a multiple of 32 and a workspace");
    KVA_REQUIRE(window >= 0 && keep_first >= 0, "latent_attention_mfma: negative window or kept first positions");
    if (window == 0) keep_first = 0;
    if (num_items == 0) return KVA_OK;
    dim3 grid(num_items, splits), block(KVA_WAVE);
    bool done = false;
#define LAUNCH_ONE(NDT, NKS)                                                                                   \
    if (!done && rank == NDT * 16 && key_dim == NKS * 32) {                                                    \
        auto kernel = (4 * NDT + 8 * NKS > 160) ? latent_attention_mfma_wide_kernel<NDT, NKS>                  \
                                                : latent_attention_mfma_kernel<NDT, NKS>;                      \
        hipLaunchKernelGGL(kernel, grid, block, 0, stream, (bf16_t *)out,                                      \
                           part_o, part_ml, (const bf16_t *)q, (const bf16_t *)cache, (const bf16_t *)cache_t, \
                           block_table, max_blocks, item_entry, item_row0, entry_seat, entry_q_start,          \
                           entry_start_pos, heads, page_size, scale, window, keep_first, sinks, splits,        \
                           per_split);                                                                         \
        done = true;                                                                                           \
    }
    LAT_INSTANCES(LAUNCH_ONE)
#undef LAUNCH_ONE
    KVA_CHECK_LAUNCH("latent_attention_mfma");
    if (splits > 1) {
        hipLaunchKernelGGL(latent_merge_kernel, dim3(total_rows), dim3(256), 0, stream, (bf16_t *)out, part_o, part_ml,
                           sinks, heads, rank, splits);
        KVA_CHECK_LAUNCH("latent_merge");
    }
    return KVA_OK;
}


// ---- grouped-query attention with the same options ---------------------------------------------
//
// The kernel above over the paged K / V^T arrays of ordinary attention (kv_layout.h), for what the
// tuned kernels of attention_mfma.hip do not take: chunks of positions that see only each other,
// a window that keeps a request's first
// positions visible, a sink per head, values of another size than the keys.  Rows of a tile are
// (token, query head of the kv head's group) pairs, row = token_in_entry * G + head_in_group; one
// wavefront per (item, kv head, key range).  D = 32 NKS key elements, DV = 16 NDT value elements.
template <int NDT, int NKS, int RT>
__global__ void __launch_bounds__(KVA_WAVE)
gqa_attention_rows_kernel(bf16_t *__restrict__ out, float *__restrict__ part_o, float *__restrict__ part_ml,
                          const bf16_t *__restrict__ q, int q_stride, const bf16_t *__restrict__ k_cache,
                          const bf16_t *__restrict__ v_cache, const int *__restrict__ block_table, int max_blocks,
                          const int *__restrict__ item_entry, const int *__restrict__ item_row0,
                          const int *__restrict__ entry_seat, const int *__restrict__ entry_q_start,
                          const int *__restrict__ entry_start_pos, int heads, int kv_heads, int page_size,
                          float scale, int window, int keep_first, int chunk, const float *__restrict__ sinks,
                          int splits, int per_split) {
    // RT tiles of 16 rows share every key and value fragment the wavefront loads (prompt portions:
    // half the loads a product with RT = 2)
    constexpr int DV = NDT * 16, D = NKS * 32;
    const int lane = threadIdx.x, r = lane & 15, g = lane >> 4;
    const int item = blockIdx.x, kvh = blockIdx.y / splits, split = blockIdx.y % splits;
    const int group = heads / kv_heads;
    const int e = item_entry[item], row0 = item_row0[item];
    const int q_start = entry_q_start[e], q_len = entry_q_start[e + 1] - q_start;
    const int start_pos = entry_start_pos[e];
    const int *bt = block_table + (size_t)entry_seat[e] * max_blocks;
    const int rows = q_len * group;
    if (row0 >= rows) return;
    const int last_row = min(row0 + 16 * RT - 1, rows - 1);
    const int item_hi = start_pos + last_row / group;
    const int pos_lo = start_pos + row0 / group;
    const int item_lo = kva_first_visible(pos_lo, window, chunk);
    const int hi_lo = kva_first_visible(item_hi, window, chunk);     // where the last row's window (or chunk) starts
    int my_pos[RT], my_lo[RT], my_head[RT];
    bool row_valid[RT];
    size_t my_token[RT];
    Frag8 qf[RT][NKS];
    f32x4 o[RT][NDT];
    float m[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int row = min(row0 + 16 * rt + r, rows - 1);
        row_valid[rt] = row0 + 16 * rt + r < rows;
        my_pos[rt] = start_pos + row / group;
        my_head[rt] = kvh * group + row % group;
        my_lo[rt] = kva_first_visible(my_pos[rt], window, chunk);
        my_token[rt] = (size_t)q_start + row / group;
        const bf16_t *qrow = q + my_token[rt] * q_stride + (size_t)my_head[rt] * D + 8 * g;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) qf[rt][ks].u4 = *reinterpret_cast<const uint4 *>(qrow + 32 * ks);
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) o[rt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        m[rt] = -INFINITY;
        l[rt] = 0.f;
    }
    const float scale2 = scale * LAT_LOG2E;

    int k_begin = 0, k_end = item_hi + 1;
    if (splits > 1) {
        k_begin = split * per_split;
        k_end = min(k_end, k_begin + per_split);
    }
    if (keep_first == 0 && item_lo > k_begin) k_begin = min(item_lo & ~31, k_end);     // nothing in front is visible
    for (int kstart = k_begin & ~31; kstart < k_end; kstart += 32) {
        if (kstart + 32 <= item_lo && kstart >= keep_first) continue;
        int page[2];
        bool mapped[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key0 = kstart + 16 * t;
            const int p = key0 <= item_hi ? bt[key0 / page_size] : -1;
            mapped[t] = p >= 0;
            page[t] = p >= 0 ? p : 0;
        }
        // every load of the block is asked for before the first product
        Frag8 kf[2][NKS], vv[NDT];
        uint2 keep[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int key = kstart + 16 * t + r;
            // K pages are [D / 8][page_size][8]: chunk 4 ks + g of key `key`
            const bf16_t *kp = k_cache + ((size_t)page[t] * kv_heads + kvh) * page_size * D +
                               ((size_t)g * page_size + key % page_size) * 8;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) kf[t][ks].u4 = *reinterpret_cast<const uint4 *>(kp + (size_t)ks * 4 * page_size * 8);
            // values: lane (element r of a tile, group g) takes keys 4 g .. 4 g + 3 of the 16-key tile
            const int key0 = kstart + 16 * t + 4 * g;
            int n = min(item_hi + 1, k_end) - key0;
            if (!mapped[t] || key0 + 4 <= k_begin) n = 0;
            keep[t] = keep_first_keys(make_uint2(~0u, ~0u), n);
            if (key0 < k_begin && n > 0) {
                const uint2 head = keep_first_keys(make_uint2(~0u, ~0u), k_begin - key0);
                keep[t].x &= ~head.x; keep[t].y &= ~head.y;
            }
            const bf16_t *vrow = v_cache + (((size_t)page[t] * kv_heads + kvh) * DV + r) * page_size + key0 % page_size;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt) vv[dt].u2[t] = *reinterpret_cast<const uint2 *>(vrow + (size_t)dt * 16 * page_size);
        }
        __builtin_amdgcn_sched_barrier(0);
        // a block that every row of the item sees whole needs no mask (wave-uniform)
        const bool whole = mapped[0] && mapped[1] && kstart >= k_begin && kstart + 32 <= k_end && kstart + 31 <= pos_lo &&
                           (kstart >= hi_lo || kstart + 32 <= keep_first);
        Frag8 pf[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            f32x4 s[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks)
                    s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][ks].v, qf[rt][ks].v, s[t], 0, 0, 0);
            }
            float sv[8], mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float x = s[t][i] * scale2;
                    if (!whole) {
                        const int key = kstart + 16 * t + 4 * g + i;
                        const bool vis = row_valid[rt] && mapped[t] && key <= my_pos[rt] &&
                                         (key >= my_lo[rt] || key < keep_first) && key >= k_begin && key < k_end;
                        x = vis ? x : -INFINITY;
                    }
                    sv[t * 4 + i] = x;
                    mx = fmaxf(mx, x);
                }
            const float bm = quad_rows_max(mx);
            if (__builtin_amdgcn_ballot_w64(bm > m[rt]) != 0) {       // the maximum moved: re-base l and O
                const float m_new = fmaxf(m[rt], bm);
                const float corr = __builtin_amdgcn_exp2f(m[rt] - ((m_new == -INFINITY) ? 0.f : m_new));
                l[rt] *= corr;
#pragma unroll
                for (int dt = 0; dt < NDT; ++dt) {
                    o[rt][dt][0] *= corr; o[rt][dt][1] *= corr; o[rt][dt][2] *= corr; o[rt][dt][3] *= corr;
                }
                m[rt] = m_new;
            }
            const float ref = (m[rt] == -INFINITY) ? 0.f : m[rt];
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                const float p0 = __builtin_amdgcn_exp2f(sv[j] - ref), p1 = __builtin_amdgcn_exp2f(sv[j + 1] - ref);
                l[rt] += p0 + p1;
                pf[rt].p2[j / 2] = pack_bf16(p0, p1);
            }
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            Frag8 v = vv[dt];
            v.u2[0].x &= keep[0].x; v.u2[0].y &= keep[0].y;
            v.u2[1].x &= keep[1].x; v.u2[1].y &= keep[1].y;
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v.v, pf[rt].v, o[rt][dt], 0, 0, 0);
        }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        float lsum = quad_rows_sum(l[rt]);
        if (!row_valid[rt]) continue;
        const size_t my_global = my_token[rt] * heads + my_head[rt];   // row of the output, of the partial results
        if (splits > 1) {
            float *po = part_o + (my_global * splits + split) * DV + 4 * g;
#pragma unroll
            for (int dt = 0; dt < NDT; ++dt)
                *reinterpret_cast<float4 *>(po + 16 * dt) = make_float4(o[rt][dt][0], o[rt][dt][1], o[rt][dt][2], o[rt][dt][3]);
            if (g == 0) {
                part_ml[(my_global * splits + split) * 2] = m[rt];
                part_ml[(my_global * splits + split) * 2 + 1] = lsum;
            }
            continue;
        }
        float mul = 1.f;
        if (sinks) {
            const float sk = sinks[my_head[rt]] * LAT_LOG2E, m_new = fmaxf(m[rt], sk);
            const float corr = __builtin_amdgcn_exp2f(m[rt] - m_new);
            lsum = lsum * corr + __builtin_amdgcn_exp2f(sk - m_new);
            mul = corr;
        }
        mul /= lsum;
        bf16_t *orow = out + my_global * DV + 4 * g;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
            Frag4 w;
            w.h[0] = float_to_bf16_bits(o[rt][dt][0] * mul); w.h[1] = float_to_bf16_bits(o[rt][dt][1] * mul);
            w.h[2] = float_to_bf16_bits(o[rt][dt][2] * mul); w.h[3] = float_to_bf16_bits(o[rt][dt][3] * mul);
            *reinterpret_cast<uint2 *>(orow + 16 * dt) = w.u2;
        }
    }
}

// (value size / 16, key size / 32) pairs with an instance
#define GQA_ROWS_INSTANCES(X) X(2, 1) X(4, 1) X(2, 2) X(4, 2) X(8, 2) X(6, 3) X(4, 4) X(8, 4) X(12, 6) X(16, 8)

extern "C" int kva_attention_rows_mfma_supported(int head_dim, int value_dim, int page_size) {
    if (page_size <= 0 || page_size % 16) return 0;
#define CHECK_ONE(NDT, NKS) if (value_dim == NDT * 16 && head_dim == NKS * 32) return 1;
    GQA_ROWS_INSTANCES(CHECK_ONE)
#undef CHECK_ONE
    return 0;
}

extern "C" int kva_attention_rows_mfma(void *out, float *part_o, float *part_ml, const void *q, int q_stride,
                                       const void *k_cache, const void *v_cache, const int *block_table,
                                       int max_blocks, const int *item_entry, const int *item_row0,
                                       const int *entry_seat, const int *entry_q_start, const int *entry_start_pos,
                                       int num_items, int total_rows, int heads, int kv_heads, int head_dim,
                                       int value_dim, int page_size, float scale, int window, int keep_first,
                                       int chunk, const float *sinks, int splits, int per_split, int row_tiles,
                                       hipStream_t stream) {
    KVA_REQUIRE(kva_attention_rows_mfma_supported(head_dim, value_dim, page_size),
                "attention_rows_mfma: no instance for keys of %d, values of %d, pages of %d", head_dim, value_dim, page_size);
    KVA_REQUIRE(num_items >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && max_blocks > 0 && total_rows >= 0,
                "attention_rows_mfma: bad sizes");
    KVA_REQUIRE(q_stride % 8 == 0 && q_stride >= heads * head_dim, "attention_rows_mfma: query row stride %d", q_stride);
    KVA_REQUIRE(splits >= 1 && (long long)splits * kv_heads <= 65535 &&
                    (splits == 1 || (per_split > 0 && per_split % 32 == 0 && part_o && part_ml)),
                "attention_rows_mfma: key ranges need a length that is a multiple of 32 and a workspace");
    KVA_REQUIRE(window >= 0 && keep_first >= 0 && chunk >= 0 && !(window > 0 && chunk > 0),
                "attention_rows_mfma: negative window, kept first positions or chunk, or a window together with chunks");
    KVA_REQUIRE(row_tiles == 1 || (row_tiles == 2 && value_dim <= 128 && head_dim <= 128),
                "attention_rows_mfma: one row tile an item, or two for heads up to 128");
    if (window == 0) keep_first = 0;
    if (num_items == 0) return KVA_OK;
    dim3 grid(num_items, kv_heads * splits), block(KVA_WAVE);
    bool done = false;
#define LAUNCH_ONE(NDT, NKS)                                                                                    \
    if (!done && value_dim == NDT * 16 && head_dim == NKS * 32) {                                               \
        auto kernel = gqa_attention_rows_kernel<NDT, NKS, 1>;                                                    \
        if constexpr (NDT <= 8 && NKS <= 4) {                                                                    \
            if (row_tiles == 2) kernel = gqa_attention_rows_kernel<NDT, NKS, 2>;                                 \
        }                                                                                                        \
        hipLaunchKernelGGL(kernel, grid, block, 0, stream, (bf16_t *)out, part_o,                                \
                           part_ml, (const bf16_t *)q, q_stride, (const bf16_t *)k_cache,                        \
                           (const bf16_t *)v_cache, block_table, max_blocks, item_entry, item_row0, entry_seat,  \
                           entry_q_start, entry_start_pos, heads, kv_heads, page_size, scale, window,            \
                           keep_first, chunk, sinks, splits, per_split);                                                \
        done = true;                                                                                             \
    }
    GQA_ROWS_INSTANCES(LAUNCH_ONE)
#undef LAUNCH_ONE
    KVA_CHECK_LAUNCH("attention_rows_mfma");
    if (splits > 1) {
        hipLaunchKernelGGL(latent_merge_kernel, dim3(total_rows), dim3(256), 0, stream, (bf16_t *)out, part_o, part_ml,
                           sinks, heads, value_dim, splits);
        KVA_CHECK_LAUNCH("attention_rows_merge");
    }
    return KVA_OK;
}
