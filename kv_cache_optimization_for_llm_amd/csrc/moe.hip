// A routed feed-forward (mixture of experts) whose work stays on the device from the router's
// logits to the weighted sum: no count of tokens per expert ever reaches the host, so the whole
// layer can be captured into a graph.
//
//  * kva_moe_route:  scores = softmax(logits) over all router outputs; the `top` largest of
//    scores + correction are chosen; their weights are the plain scores (optionally renormalised).
//    Or (`over_chosen`) the largest logits are chosen and the weights are the softmax over them alone.
//  * kva_moe_align:  the (token, choice) slots of real experts sorted by expert into a list padded
//    so that every tile of 16 rows belongs to one expert (`sorted_slot`, -1 = padding), with the
//    expert of every tile (`tile_expert`, -1 = unused tile).
//  * kva_moe_expert_rows: one product per tile against its expert's matrix.  Mode 0 ("up"): rows of
//    x gathered by slot / top, activation applied (a gated expert: act(gate) * up, its gate and up rows
//    interleaved in one matrix), written at the sorted position.  Mode 1 ("down"):
//    rows at the sorted position, times the slot's routing weight, written at the slot (fp32).
//    bf16 with K % 32 == 0 runs on the matrix cores, everything else (fp32 too) on a plain tiled
//    kernel that adds k ascending.
//  * kva_moe_combine: out[t] = sum over the token's choices of the slot's row, or, for a router
//    output past the real experts (an identity expert), weight * x[t].
//
// A row's result depends on that row and its expert's matrix only, never on which other rows
// share its tile: the same token gives the same numbers in any batch.
#include "common.h"
#include "attention_frag.h"
#include <math.h>

#define MOE_TILE 16
#define MOE_MAX_EXPERTS 1024
#define MOE_ROUTE_PER_LANE 8

__device__ inline float moe_activate(float z, int act) {
    if (act == 3) return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));       // exact gelu
    return kva_activate(z, act);
}

// ---- router ------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
moe_route_kernel(int *__restrict__ idx, float *__restrict__ wgt, const float *__restrict__ logits,
                 const float *__restrict__ correction, int tokens, int outputs, int top, int renormalise,
                 int over_chosen, int sigmoid_scores, int groups, int keep_groups, int group_top, float weight_scale,
                 float sum_eps, int logits_stride) {
    __shared__ float choice_s[4][KVA_WAVE * MOE_ROUTE_PER_LANE];
    const int lane = threadIdx.x % KVA_WAVE;
    const int t = blockIdx.x * (blockDim.x / KVA_WAVE) + threadIdx.x / KVA_WAVE;
    if (t >= tokens) return;
    float *choice = choice_s[threadIdx.x / KVA_WAVE];
    float s[MOE_ROUTE_PER_LANE], ch[MOE_ROUTE_PER_LANE];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j) {
        const int e = lane + j * KVA_WAVE;
        s[j] = e < outputs ? logits[(size_t)t * logits_stride + e] : -INFINITY;
        mx = fmaxf(mx, s[j]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j) {
        const int e = lane + j * KVA_WAVE;
        s[j] = e < outputs ? expf(s[j] - mx) : 0.f;
        sum += s[j];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j) {
        const int e = lane + j * KVA_WAVE;
        if (over_chosen) {
            // the logits themselves are compared, and the weights are a softmax over the chosen ones
            // alone: exp(logit - max) here, divided by the chosen ones' sum below
            ch[j] = e < outputs ? logits[(size_t)t * logits_stride + e] + (correction ? correction[e] : 0.f) : -INFINITY;
        } else {
            // scores: the softmax over all outputs, or every output's own sigmoid
            s[j] = sigmoid_scores ? (e < outputs ? 1.f / (1.f + expf(-logits[(size_t)t * logits_stride + e])) : 0.f) : s[j] / sum;
            ch[j] = e < outputs ? s[j] + (correction ? correction[e] : 0.f) : -INFINITY;
        }
    }
    if (groups > 1) {
        // Outputs form `groups` equal runs of neighbours.  A group's score is the sum of its `group_top`
        // largest choice scores; only outputs of the `keep_groups` best groups (of equal ones the lowest
        // index) can be chosen: the others' choice scores become -inf.  Lane g takes group g.
        const int per = outputs / groups;
#pragma unroll
        for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j)
            if (lane + j * KVA_WAVE < outputs) choice[lane + j * KVA_WAVE] = ch[j];
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
        float gs = -INFINITY;
        if (lane < groups) {
            gs = 0.f;
            unsigned long long taken = 0ull;            // (a group holds at most 64 outputs when it is scored this way; larger ones below)
            for (int k = 0; k < group_top && k < per; ++k) {
                float bv = -INFINITY;
                int bi = -1;
                for (int i = 0; i < per; ++i) {
                    const bool used = i < 64 ? ((taken >> i) & 1ull) != 0ull : false;
                    const float v = choice[lane * per + i];
                    if (!used && (bi < 0 || v > bv)) { bv = v; bi = i; }
                }
                if (bi >= 0 && bi < 64) taken |= 1ull << bi;
                gs += bv;
            }
        }
        unsigned long long allowed = 0ull;
        for (int k = 0; k < keep_groups; ++k) {
            float bv = gs;
            int bg = lane < groups && !((allowed >> lane) & 1ull) ? lane : 0x7fffffff;
            if (bg == 0x7fffffff) bv = -INFINITY;
#pragma unroll
            for (int off = KVA_WAVE / 2; off > 0; off >>= 1) {
                const float ov = __shfl_xor(bv, off, KVA_WAVE);
                const int og = __shfl_xor(bg, off, KVA_WAVE);
                if (og != 0x7fffffff && (bg == 0x7fffffff || ov > bv || (ov == bv && og < bg))) { bv = ov; bg = og; }
            }
            if (bg != 0x7fffffff) allowed |= 1ull << bg;
        }
#pragma unroll
        for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j) {
            const int e = lane + j * KVA_WAVE;
            if (e < outputs && !((allowed >> (e / per)) & 1ull)) ch[j] = -INFINITY;
        }
    }
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        // the largest remaining choice score; of equal ones the lowest index
        float bv = -INFINITY, bs = 0.f;
        int be = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j) {
            const int e = lane + j * KVA_WAVE;
            if (e < outputs && (ch[j] > bv || (ch[j] == bv && e < be))) { bv = ch[j]; be = e; bs = s[j]; }
        }
#pragma unroll
        for (int off = KVA_WAVE / 2; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, KVA_WAVE), os = __shfl_xor(bs, off, KVA_WAVE);
            const int oe = __shfl_xor(be, off, KVA_WAVE);
            if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; bs = os; }
        }
#pragma unroll
        for (int j = 0; j < MOE_ROUTE_PER_LANE; ++j)
            if (lane + j * KVA_WAVE == be) ch[j] = -INFINITY;
        total += bs;
        if (lane == 0) {
            idx[(size_t)t * top + k] = be;
            wgt[(size_t)t * top + k] = bs;
        }
    }
    if (lane == 0) {
        if (renormalise || over_chosen)
            for (int k = 0; k < top; ++k) wgt[(size_t)t * top + k] = wgt[(size_t)t * top + k] / (total + sum_eps) * weight_scale;
        else if (weight_scale != 1.f)
            for (int k = 0; k < top; ++k) wgt[(size_t)t * top + k] *= weight_scale;
    }
}

extern "C" int kva_moe_route(int *idx, float *wgt, const float *logits, const float *correction, int tokens,
                             int outputs, int top, int renormalise, int over_chosen, int sigmoid_scores, int groups,
                             int keep_groups, int group_top, float weight_scale, float sum_eps, int logits_stride,
                             hipStream_t stream) {
    // logits_stride: elements between two tokens' rows of logits (the logits may be the first columns of a wider product)
    KVA_REQUIRE(logits_stride >= outputs, "moe_route: a row of logits holds at least the %d outputs", outputs);
    KVA_REQUIRE(groups >= 1 && groups <= KVA_WAVE && outputs % groups == 0 && keep_groups >= 1 && keep_groups <= groups &&
                    group_top >= 1,
                "moe_route: %d groups (at most %d, dividing the %d outputs) of which %d are kept", groups, KVA_WAVE, outputs,
                keep_groups);
    KVA_REQUIRE(groups == 1 || (outputs / groups <= 64 && top <= keep_groups * (outputs / groups)),
                "moe_route: groups of at most 64 outputs, and enough outputs in the kept groups for top %d", top);
    KVA_REQUIRE(!(sigmoid_scores && over_chosen), "moe_route: sigmoid scores exclude the softmax over the chosen logits");
    KVA_REQUIRE(idx && wgt && logits && tokens >= 0, "moe_route: missing operand");
    KVA_REQUIRE(outputs > 0 && outputs <= KVA_WAVE * MOE_ROUTE_PER_LANE, "moe_route: %d router outputs (at most %d)",
                outputs, KVA_WAVE * MOE_ROUTE_PER_LANE);
    KVA_REQUIRE(top > 0 && top <= outputs, "moe_route: top %d of %d", top, outputs);
    if (tokens == 0) return KVA_OK;
    hipLaunchKernelGGL(moe_route_kernel, dim3((tokens + 3) / 4), dim3(256), 0, stream, idx, wgt, logits, correction,
                       tokens, outputs, top, renormalise, over_chosen, sigmoid_scores, groups, keep_groups, group_top,
                       weight_scale, sum_eps, logits_stride);
    KVA_CHECK_LAUNCH("moe_route");
    return KVA_OK;
}

// ---- slots sorted by expert --------------------------------------------------------------
__global__ void __launch_bounds__(1024)
moe_align_kernel(int *__restrict__ sorted_slot, int *__restrict__ tile_expert, const int *__restrict__ idx, int slots,
                 int experts, int capacity, int max_tiles) {
    __shared__ int count[MOE_MAX_EXPERTS], start[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
    for (int p = threadIdx.x; p < capacity; p += blockDim.x) sorted_slot[p] = -1;
    for (int i = threadIdx.x; i < max_tiles; i += blockDim.x) tile_expert[i] = -1;
    __syncthreads();
    for (int s = threadIdx.x; s < slots; s += blockDim.x) {
        const int e = idx[s];
        if (e >= 0 && e < experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            start[e] = at;
            const int tiles = (count[e] + MOE_TILE - 1) / MOE_TILE;
            for (int i = 0; i < tiles; ++i) tile_expert[at / MOE_TILE + i] = e;
            at += tiles * MOE_TILE;
            count[e] = 0;               // from here on: the next free place of the expert's run
        }
    }
    __syncthreads();
    for (int s = threadIdx.x; s < slots; s += blockDim.x) {
        const int e = idx[s];
        if (e >= 0 && e < experts) sorted_slot[start[e] + atomicAdd(&count[e], 1)] = s;
    }
}

extern "C" int kva_moe_align(int *sorted_slot, int *tile_expert, const int *idx, int slots, int experts, int capacity,
                             int max_tiles, hipStream_t stream) {
    KVA_REQUIRE(sorted_slot && tile_expert && idx, "moe_align: missing operand");
    KVA_REQUIRE(experts > 0 && experts <= MOE_MAX_EXPERTS, "moe_align: %d experts (at most %d)", experts, MOE_MAX_EXPERTS);
    KVA_REQUIRE(capacity == max_tiles * MOE_TILE && capacity >= slots + experts * (MOE_TILE - 1),
                "moe_align: a list of %d places cannot hold %d slots of %d experts in tiles of %d", capacity, slots,
                experts, MOE_TILE);
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), 0, stream, sorted_slot, tile_expert, idx, slots, experts,
                       capacity, max_tiles);
    KVA_CHECK_LAUNCH("moe_align");
    return KVA_OK;
}

// ---- one product per tile ------------------------------------------------------------------
struct MoeRows {
    const int *sorted_slot, *tile_expert;
    const float *slot_weight;       // mode 1
    int top, N, K, mode, act;
    int gated;                      // mode 0: rows 2 j and 2 j + 1 of the matrix are output j's gate and up rows
    float limit;                    // activation 4 (clamped swish): gate and up are cut off at this value
};

// mode 0 of a gated expert: outputs n (even) and n + 1 of the product are one output of the layer
__device__ inline void moe_store_gated(const MoeRows &a, void *out, int out_dtype, int place, int n, float gate, float up) {
    const float v = a.act == 4 ? kva_gated_activate(gate, up, KVA_ACT_SWISH_CLAMPED, a.limit) : moe_activate(gate, a.act) * up;
    const size_t at = (size_t)place * (a.N / 2) + n / 2;
    if (out_dtype == KVA_BF16) reinterpret_cast<uint16_t *>(out)[at] = float_to_bf16_bits(v);
    else reinterpret_cast<float *>(out)[at] = v;
}

__device__ inline void moe_store(const MoeRows &a, void *out, int out_dtype, int place, int slot, int n, float v) {
    if (a.mode == 0) {
        v = moe_activate(v, a.act);
        if (out_dtype == KVA_BF16) reinterpret_cast<uint16_t *>(out)[(size_t)place * a.N + n] = float_to_bf16_bits(v);
        else reinterpret_cast<float *>(out)[(size_t)place * a.N + n] = v;
    } else {
        reinterpret_cast<float *>(out)[(size_t)slot * a.N + n] = v * a.slot_weight[slot];
    }
}

// plain: a workgroup takes a tile of 16 rows and 64 outputs; thread (row, cx) 4 neighbouring outputs
template <typename T>
__global__ void __launch_bounds__(256)
moe_expert_rows_kernel(MoeRows a, void *__restrict__ out, int out_dtype, const T *__restrict__ x,
                       const T *__restrict__ w) {
    __shared__ float xs[MOE_TILE][33], ws[64][33];
    const int tile = blockIdx.y, e = a.tile_expert[tile];
    if (e < 0) return;
    const int n0 = blockIdx.x * 64, row = threadIdx.x / 16, cx = threadIdx.x % 16;
    const int place = tile * MOE_TILE + row, slot = a.sorted_slot[place];
    const T *wm = w + (size_t)e * a.N * a.K;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < a.K; k0 += 32) {
        __syncthreads();
        for (int i = threadIdx.x; i < MOE_TILE * 32; i += 256) {
            const int rr = i / 32, kk = k0 + i % 32;
            const int sl = a.sorted_slot[tile * MOE_TILE + rr];
            const size_t src = a.mode == 0 ? (size_t)(sl < 0 ? 0 : sl / a.top) : (size_t)(tile * MOE_TILE + rr);
            xs[rr][i % 32] = (kk < a.K && sl >= 0) ? to_float(x[src * a.K + kk]) : 0.f;
        }
        for (int i = threadIdx.x; i < 64 * 32; i += 256) {
            const int nn = n0 + i / 32, kk = k0 + i % 32;
            ws[i / 32][i % 32] = (nn < a.N && kk < a.K) ? to_float(wm[(size_t)nn * a.K + kk]) : 0.f;
        }
        __syncthreads();
        for (int kk = 0; kk < 32; ++kk) {
            const float xv = xs[row][kk];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] += xv * ws[4 * cx + j][kk];
        }
    }
    if (slot < 0) return;
    if (a.gated) {
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
            const int n = n0 + 4 * cx + j;
            if (n + 1 < a.N) moe_store_gated(a, out, out_dtype, place, n, acc[j], acc[j + 1]);
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + 4 * cx + j;
        if (n < a.N) moe_store(a, out, out_dtype, place, slot, n, acc[j]);
    }
}

// matrix cores: a workgroup takes RT tiles of 16 rows and NT tiles of 16 outputs; out^T[n, t] =
// W[e][n, :] . x[t, :]; operands straight from memory, 16 bytes a lane and product.  Its four
// wavefronts take a quarter of K each (the same quarters whatever NT, RT and the batch are) and the
// first adds the four partial results up in a fixed order: with few tiles - decoded tokens - there are
// four times as many wavefronts streaming the experts' matrices.  Row tiles of one expert (the list is
// sorted by expert, so neighbours mostly are) share what is loaded of its matrix; a group of tiles
// that spans two experts is walked tile by tile.
template <int NT, int RT>
__device__ inline void moe_tiles_product(const MoeRows &a, void *__restrict__ out, int out_dtype,
                                         const bf16_t *__restrict__ x, const bf16_t *__restrict__ w, int first_tile,
                                         int e, int n_first, float (*red)[KVA_WAVE][4]) {
    const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE, r = lane & 15, g = lane >> 4;
    int place[RT], slot[RT];
    const bf16_t *xrow[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        place[rt] = (first_tile + rt) * MOE_TILE + r;
        slot[rt] = a.sorted_slot[place[rt]];
        const size_t src = a.mode == 0 ? (size_t)(slot[rt] < 0 ? 0 : slot[rt] / a.top) : (size_t)place[rt];
        xrow[rt] = x + src * a.K + 8 * g;
    }
    const bf16_t *wrow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
        wrow[nt] = w + ((size_t)e * a.N + min(n_first + 16 * nt + r, a.N - 1)) * a.K + 8 * g;
    f32x4 acc[NT][RT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[nt][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int steps = a.K / 32, per = (steps + 3) / 4;
    const int s0 = wave * per, s1 = min(steps, s0 + per);
#pragma unroll 2
    for (int s = s0; s < s1; ++s) {
        const int k0 = 32 * s;
        Frag8 xf[RT], wf[NT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) xf[rt].u4 = *reinterpret_cast<const uint4 *>(xrow[rt] + k0);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wf[nt].u4 = *reinterpret_cast<const uint4 *>(wrow[nt] + k0);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
                acc[nt][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[nt].v, xf[rt].v, acc[nt][rt], 0, 0, 0);
    }
    __syncthreads();                 // whoever still reads the partial results of the call before is done
    if (wave > 0)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[((wave - 1) * NT + nt) * RT + rt][lane][i] = acc[nt][rt][i];
    __syncthreads();
    if (wave > 0) return;
    // lane (row r, group g) holds outputs n0 + 4 g .. + 3 of its row
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (slot[rt] < 0) continue;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float v[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                v[i] = ((acc[nt][rt][i] + red[(0 * NT + nt) * RT + rt][lane][i]) + red[(1 * NT + nt) * RT + rt][lane][i])
                       + red[(2 * NT + nt) * RT + rt][lane][i];
            const int n = n_first + 16 * nt + 4 * g;
            if (a.gated) {
                if (n + 1 < a.N) moe_store_gated(a, out, out_dtype, place[rt], n, v[0], v[1]);
                if (n + 3 < a.N) moe_store_gated(a, out, out_dtype, place[rt], n + 2, v[2], v[3]);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < a.N) moe_store(a, out, out_dtype, place[rt], slot[rt], n + i, v[i]);
            }
        }
    }
}

template <int NT, int RT>
__global__ void __launch_bounds__(256)
moe_expert_rows_mfma_kernel(MoeRows a, void *__restrict__ out, int out_dtype, const bf16_t *__restrict__ x,
                            const bf16_t *__restrict__ w, int max_tiles) {
    __shared__ float red[3 * NT * RT][KVA_WAVE][4];
    const int first = blockIdx.y * RT, n_first = blockIdx.x * 16 * NT;
    const int e0 = a.tile_expert[first];
    bool same = e0 >= 0;
#pragma unroll
    for (int rt = 1; rt < RT; ++rt) same = same && first + rt < max_tiles && a.tile_expert[first + rt] == e0;
    if (same) {
        moe_tiles_product<NT, RT>(a, out, out_dtype, x, w, first, e0, n_first, red);
        return;
    }
    for (int rt = 0; rt < RT; ++rt) {
        const int e = first + rt < max_tiles ? a.tile_expert[first + rt] : -1;
        if (e >= 0) moe_tiles_product<NT, 1>(a, out, out_dtype, x, w, first + rt, e, n_first, red);
    }
}

extern "C" int kva_moe_expert_rows(void *out, int out_dtype, const void *x, const void *w, int dtype,
                                   const int *sorted_slot, const int *tile_expert, const float *slot_weight,
                                   int max_tiles, int top, int N, int K, int mode, int act, int gated, float limit,
                                   hipStream_t stream) {
    KVA_REQUIRE(act != 4 || gated, "moe_expert_rows: the clamped activation is a gated one");
    KVA_REQUIRE(!gated || (mode == 0 && N % 2 == 0), "moe_expert_rows: gate and up rows come in pairs, in the first product");
    KVA_REQUIRE(out && x && w && sorted_slot && tile_expert, "moe_expert_rows: missing operand");
    KVA_REQUIRE(mode == 0 || (mode == 1 && slot_weight && out_dtype == KVA_F32),
                "moe_expert_rows: mode 1 writes fp32 rows times a weight per slot");
    KVA_REQUIRE(mode == 1 || out_dtype == dtype, "moe_expert_rows: mode 0 writes rows of the operands' type");
    KVA_REQUIRE(N > 0 && K > 0 && top > 0 && act >= 0 && act <= 4, "moe_expert_rows: bad sizes or activation");
    KVA_REQUIRE(max_tiles >= 0 && max_tiles <= 65535, "moe_expert_rows: %d tiles are too many for one launch", max_tiles);
    if (max_tiles == 0) return KVA_OK;
    MoeRows a{sorted_slot, tile_expert, slot_weight, top, N, K, mode, act, gated, limit};
    if (dtype == KVA_BF16 && K % 32 == 0) {
        // few tiles: 16 outputs a workgroup, so that enough of them stream the matrices; many: 64 outputs and
        // four row tiles, which share what they load
        if ((long long)max_tiles * ((N + 15) / 16) <= 8192)
            hipLaunchKernelGGL((moe_expert_rows_mfma_kernel<1, 1>), dim3((N + 15) / 16, max_tiles), dim3(256), 0, stream, a,
                               out, out_dtype, (const bf16_t *)x, (const bf16_t *)w, max_tiles);
        else
            hipLaunchKernelGGL((moe_expert_rows_mfma_kernel<4, 4>), dim3((N + 63) / 64, (max_tiles + 3) / 4), dim3(256), 0,
                               stream, a, out, out_dtype, (const bf16_t *)x, (const bf16_t *)w, max_tiles);
    } else if (dtype == KVA_BF16) {
        hipLaunchKernelGGL(moe_expert_rows_kernel<bf16_t>, dim3((N + 63) / 64, max_tiles), dim3(256), 0, stream, a, out,
                           out_dtype, (const bf16_t *)x, (const bf16_t *)w);
    } else if (dtype == KVA_F32) {
        hipLaunchKernelGGL(moe_expert_rows_kernel<float>, dim3((N + 63) / 64, max_tiles), dim3(256), 0, stream, a, out,
                           out_dtype, (const float *)x, (const float *)w);
    } else KVA_REQUIRE(false, "moe_expert_rows: unsupported dtype %d", dtype);
    KVA_CHECK_LAUNCH("moe_expert_rows");
    return KVA_OK;
}

// ---- weighted sum --------------------------------------------------------------------------
__device__ inline float moe_ld(const void *p, int dtype, size_t i) {
    return dtype == KVA_BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(p)[i])
                             : reinterpret_cast<const float *>(p)[i];
}

__global__ void __launch_bounds__(256)
moe_combine_kernel(void *__restrict__ out, const void *__restrict__ x, int dtype, const float *__restrict__ rows,
                   const int *__restrict__ idx, const float *__restrict__ wgt, const void *__restrict__ extra,
                   const float *__restrict__ extra_gate, int extra_gate_stride, int width, int top, int experts) {
    const size_t t = blockIdx.x;
    // (optional) the addend enters times sigmoid(extra_gate[t * stride]), one number a token (a column of a wider array)
    const float eg = extra && extra_gate ? 1.f / (1.f + expf(-extra_gate[t * extra_gate_stride])) : 1.f;
    if (width % 4 == 0 && ((reinterpret_cast<uintptr_t>(rows) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        // four neighbouring columns a thread, 16 bytes of every row at a time; the additions per column are
        // in the order of the scalar loop below
        for (int j = threadIdx.x * 4; j < width; j += blockDim.x * 4) {
            float acc[4] = {0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < top; ++k) {
                const size_t s = t * top + k;
                if (idx[s] < experts) {
                    const float4 r = *reinterpret_cast<const float4 *>(rows + s * width + j);
                    acc[0] += r.x; acc[1] += r.y; acc[2] += r.z; acc[3] += r.w;
                } else {
                    const float g = wgt[s];
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[e] += g * moe_ld(x, dtype, t * width + j + e);
                }
            }
            if (extra) {
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += eg * moe_ld(extra, dtype, t * width + j + e);
            }
            if (dtype == KVA_BF16) {
                const uint2 o = make_uint2((uint32_t)float_to_bf16_bits(acc[0]) | ((uint32_t)float_to_bf16_bits(acc[1]) << 16),
                                           (uint32_t)float_to_bf16_bits(acc[2]) | ((uint32_t)float_to_bf16_bits(acc[3]) << 16));
                *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(out) + t * width + j) = o;
            } else {
                *reinterpret_cast<float4 *>(reinterpret_cast<float *>(out) + t * width + j) = make_float4(acc[0], acc[1], acc[2], acc[3]);
            }
        }
        return;
    }
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const size_t s = t * top + k;
            if (idx[s] < experts) acc += rows[s * width + j];
            else acc += wgt[s] * (dtype == KVA_BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(x)[t * width + j])
                                                    : reinterpret_cast<const float *>(x)[t * width + j]);
        }
        // what an expert that every token uses returned, with weight 1
        if (extra) acc += eg * (dtype == KVA_BF16 ? bf16_bits_to_float(reinterpret_cast<const uint16_t *>(extra)[t * width + j])
                                                  : reinterpret_cast<const float *>(extra)[t * width + j]);
        if (dtype == KVA_BF16) reinterpret_cast<uint16_t *>(out)[t * width + j] = float_to_bf16_bits(acc);
        else reinterpret_cast<float *>(out)[t * width + j] = acc;
    }
}

extern "C" int kva_moe_combine(void *out, const void *x, int dtype, const float *rows, const int *idx,
                               const float *wgt, const void *extra, const float *extra_gate, int extra_gate_stride,
                               int tokens, int width, int top, int experts, hipStream_t stream) {
    KVA_REQUIRE(out && x && rows && idx && wgt && width > 0 && top > 0, "moe_combine: missing operand");
    KVA_REQUIRE(dtype == KVA_BF16 || dtype == KVA_F32, "moe_combine: unsupported dtype %d", dtype);
    if (tokens <= 0) return KVA_OK;
    hipLaunchKernelGGL(moe_combine_kernel, dim3(tokens), dim3(256), 0, stream, out, x, dtype, rows, idx, wgt, extra, extra_gate,
                       extra_gate_stride, width, top, experts);
    KVA_CHECK_LAUNCH("moe_combine");
    return KVA_OK;
}

// ---- small products with 32-bit results -------------------------------------------------------
// out[t, n] = sum_k x[t, k] * w[n, k] in fp32, for the small matrices whose results must not be rounded
// to 16 bits (a router's logits; the second half of a low-rank projection that makes decays, which
// may be finished here: bias, sigmoid, power).  x and
// w may be bf16 or fp32; every product and sum is fp32.  A workgroup takes a token: its row of x goes
// to LDS once; with a long K a wavefront takes an output and its lanes stride over K (sum by
// wavefront reduction), with a short K a thread takes an output.  The order of every sum depends on
// the sizes alone.
#define SMALL_PRODUCT_MAX_K 8192

// eight neighbouring elements from index i on (i a multiple of 8: 16 or 32 aligned bytes)
__device__ inline void moe_ld8(const void *p, int dtype, size_t i, float (&f)[8]) {
    if (dtype == KVA_BF16) {
        const uint4 v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(p) + i);
        const unsigned u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = __uint_as_float(u[j] << 16);
            f[2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
        }
    } else {
        const float4 a = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p) + i);
        const float4 b = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p) + i + 4);
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
}

// the result as it is, plus a bias, or - with decay_inv_tau > 0 - turned into a decay:
// sigmoid(z)^(1 / tau) = exp(-softplus(-z) / tau) with z = the sum plus its bias
// or - with rate_log - into exp(-exp(rate_log[n / rate_group]) softplus(z)): a decay per output whose rate
// is shared by groups of neighbouring outputs (the key channels of a head)
__device__ inline float small_product_finish(float acc, const float *bias, int n, float decay_inv_tau,
                                             const float *rate_log, int rate_group) {
    const float z = acc + (bias ? bias[n] : 0.f);
    if (rate_log) return expf(-expf(rate_log[n / rate_group]) * (fmaxf(z, 0.f) + log1pf(expf(-fabsf(z)))));
    if (decay_inv_tau <= 0.f) return z;
    const float softplus = fmaxf(-z, 0.f) + log1pf(expf(-fabsf(z)));
    return expf(-softplus * decay_inv_tau);
}

__global__ void __launch_bounds__(256)
small_product_f32_kernel(float *__restrict__ out, const void *__restrict__ x, int x_dtype, int x_stride,
                         const void *__restrict__ w, int w_dtype, int N, int K, int per_block,
                         const float *__restrict__ bias, float decay_inv_tau, const float *__restrict__ rate_log,
                         int rate_group) {
    extern __shared__ float xs[];
    const size_t t = blockIdx.x;
    const int n_lo = blockIdx.y * per_block, n_hi = min(N, n_lo + per_block);
    for (int k = threadIdx.x; k < K; k += blockDim.x) xs[k] = moe_ld(x, x_dtype, t * x_stride + k);
    __syncthreads();
    const int K8 = (K % 8 == 0) ? K : 0;          // the part read eight elements at a time
    if (K >= 128) {
        const int lane = threadIdx.x % KVA_WAVE, wave = threadIdx.x / KVA_WAVE, waves = blockDim.x / KVA_WAVE;
        for (int n = n_lo + wave; n < n_hi; n += waves) {
            float acc = 0.f;
            for (int k = 8 * lane; k < K8; k += 8 * KVA_WAVE) {
                float f[8];
                moe_ld8(w, w_dtype, (size_t)n * K + k, f);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc += xs[k + i] * f[i];
            }
            for (int k = K8 + lane; k < K; k += KVA_WAVE) acc += xs[k] * moe_ld(w, w_dtype, (size_t)n * K + k);
            acc = wave_sum(acc);
            if (lane == 0) out[t * N + n] = small_product_finish(acc, bias, n, decay_inv_tau, rate_log, rate_group);
        }
    } else {
        for (int n = n_lo + threadIdx.x; n < n_hi; n += blockDim.x) {
            float acc = 0.f;
            for (int k = 0; k < K8; k += 8) {
                float f[8];
                moe_ld8(w, w_dtype, (size_t)n * K + k, f);
#pragma unroll
                for (int i = 0; i < 8; ++i) acc += xs[k + i] * f[i];
            }
            for (int k = K8; k < K; ++k) acc += xs[k] * moe_ld(w, w_dtype, (size_t)n * K + k);
            out[t * N + n] = small_product_finish(acc, bias, n, decay_inv_tau, rate_log, rate_group);
        }
    }
}

extern "C" int kva_small_product_f32(float *out, const void *x, int x_dtype, int x_stride, const void *w, int w_dtype,
                                     int tokens, int N, int K, const float *bias, float decay_inv_tau,
                                     const float *rate_log, int rate_group, hipStream_t stream) {
    KVA_REQUIRE(!rate_log || (rate_group > 0 && N % rate_group == 0 && decay_inv_tau <= 0.f),
                "small_product_f32: rates are shared by whole groups of outputs, and exclude the other decay");
    KVA_REQUIRE(out && x && w && tokens >= 0 && N > 0, "small_product_f32: missing operand or bad sizes");
    KVA_REQUIRE(K > 0 && K <= SMALL_PRODUCT_MAX_K && x_stride >= K, "small_product_f32: K %d must lie in 1..%d", K, SMALL_PRODUCT_MAX_K);
    KVA_REQUIRE((x_dtype == KVA_BF16 || x_dtype == KVA_F32) && (w_dtype == KVA_BF16 || w_dtype == KVA_F32),
                "small_product_f32: unsupported dtype");
    if (tokens == 0) return KVA_OK;
    KVA_REQUIRE((reinterpret_cast<uintptr_t>(w) & 31) == 0, "small_product_f32: the matrix must be aligned to 32 bytes");
    const int per_block = K >= 128 ? 16 : 256;         // outputs a workgroup: four a wavefront, or one a thread
    const int blocks_y = (N + per_block - 1) / per_block;
    KVA_REQUIRE(tokens <= 0x7fffffff && blocks_y <= 65535, "small_product_f32: too many outputs");
    hipLaunchKernelGGL(small_product_f32_kernel, dim3(tokens, blocks_y), dim3(256), (size_t)K * sizeof(float), stream,
                       out, x, x_dtype, x_stride, w, w_dtype, N, K, per_block, bias, decay_inv_tau, rate_log,
                       rate_group > 0 ? rate_group : 1);
    KVA_CHECK_LAUNCH("small_product_f32");
    return KVA_OK;
}
