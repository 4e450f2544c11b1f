// The routing of a mixture of experts, on the device from the router's logits to the weighted
// sum of the experts' outputs; the host never sees a count.
//   scores    s = softmax(z) over all experts (float32)
//   choice    the `top` largest scores (the lower index wins a tie)
//   weights   the chosen scores, divided by their sum + eps where asked
//   lists     the (token, choice) pairs sorted by expert: expert e owns the sorted rows
//             row_start[e] .. row_start[e + 1] - 1, tile_start[e] counts the tiles of `tile` rows of
//             the experts before it (the grouped product's work list), sorted_token[row] is the
//             row's token and entry_row[token * top + k] the row of a token's k-th choice
//   combine   out[t] = sum_k weight[t][k] * y[entry_row[t][k]], k in the order of the choice
// A sorted row's value does not depend on where in its expert's stretch it lies, so the order in
// which the pairs of one expert arrive (atomic counters) changes no result.
#include "common.h"
#include "activations.h"

namespace lc {

constexpr int MOE_MAX_EXPERTS = 512;      // 8 a lane of the routing wave
constexpr int MOE_PER_LANE = MOE_MAX_EXPERTS / kWave;

// One wave per token.
__global__ __launch_bounds__(kWave) void moe_route_kernel(const float* __restrict__ logits, int E, int top,
                                                         int renormalise, float eps, int* __restrict__ ids,
                                                         float* __restrict__ weights) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * E;
    float s[MOE_PER_LANE];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < MOE_PER_LANE; ++i) {
        const int e = lane + kWave * i;
        s[i] = e < E ? z[e] : -INFINITY;
        m = fmaxf(m, s[i]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < MOE_PER_LANE; ++i) {
        s[i] = lane + kWave * i < E ? expf(s[i] - m) : -1.f;     // -1: no expert, below every score
        sum += fmaxf(s[i], 0.f);
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < MOE_PER_LANE; ++i)
        if (s[i] >= 0.f) s[i] = s[i] / sum;
    float picked_sum = 0.f, mine = 0.f;       // lane k keeps the k-th choice's score
    for (int k = 0; k < top; ++k) {
        float best = -1.f;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i)
            if (s[i] > best) { best = s[i]; at = lane + kWave * i; }     // a lane's experts in rising order
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, kWave);
            const int oa = __shfl_xor(at, off, kWave);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i)
            if (lane + kWave * i == at) s[i] = -1.f;
        if (lane == 0) ids[(size_t)t * top + k] = at;
        if (lane == k) mine = best;
        picked_sum += best;
    }
    const float div = renormalise ? picked_sum + eps : 1.f;
    if (lane < top) weights[(size_t)t * top + lane] = mine / div;
}

// One wave per token: the `top` largest of logits + bias (the lower index wins a tie), weighing as
// the softmax over the chosen logits alone.  `cols`: entries of a row of `logits` (>= E).
__global__ __launch_bounds__(kWave) void moe_route_logits_kernel(const float* __restrict__ logits, int cols,
                                                                const float* __restrict__ bias, int E, int top,
                                                                int* __restrict__ ids, float* __restrict__ weights) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * cols;
    float s[MOE_PER_LANE];
#pragma unroll
    for (int i = 0; i < MOE_PER_LANE; ++i) {
        const int e = lane + kWave * i;
        s[i] = e < E ? z[e] + (bias ? bias[e] : 0.f) : -INFINITY;
    }
    float first = 0.f, picked_sum = 0.f, mine = 0.f;      // lane k keeps exp(k-th chosen logit - the largest)
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i)
            if (s[i] > best) { best = s[i]; at = lane + kWave * i; }     // a lane's experts in rising order
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, kWave);
            const int oa = __shfl_xor(at, off, kWave);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i)
            if (lane + kWave * i == at) s[i] = -INFINITY;
        if (k == 0) first = best;
        const float w = expf(best - first);
        if (lane == 0) ids[(size_t)t * top + k] = at < E ? at : 0;
        if (lane == k) mine = w;
        picked_sum += w;
    }
    if (lane < top) weights[(size_t)t * top + lane] = mine / picked_sum;
}

// One wave per token: scores s = sigmoid(z); the choice goes by s + correction, the weights by s alone,
// times `scale`.  With `groups` > 1 the experts form that many equal groups of neighbours; a group's
// rank is the sum of its two largest choice scores (of its one, where a group is one expert), and only
// the experts of the `keep` best groups can be chosen: the others leave the contest whatever their
// score.  The lower index wins every tie, among groups and among experts.
__global__ __launch_bounds__(kWave) void moe_route_sigmoid_kernel(const float* __restrict__ logits,
                                                                 const float* __restrict__ correction, int E,
                                                                 int top, int groups, int keep, float scale,
                                                                 int* __restrict__ ids, float* __restrict__ weights) {
    __shared__ float choice_s[MOE_MAX_EXPERTS];
    __shared__ float score_s[MOE_MAX_EXPERTS];
    __shared__ float rank_s[MOE_MAX_EXPERTS];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * E;
    float c[MOE_PER_LANE];
#pragma unroll
    for (int i = 0; i < MOE_PER_LANE; ++i) {
        const int e = lane + kWave * i;
        c[i] = -INFINITY;
        if (e < E) {
            const float s = 1.f / (1.f + expf(-z[e]));
            score_s[e] = s;
            c[i] = s + (correction ? correction[e] : 0.f);
            choice_s[e] = c[i];
        }
    }
    __syncthreads();
    if (groups > 1) {
        const int per = E / groups;
        for (int g = lane; g < groups; g += kWave) {
            float a = -INFINITY, b = -INFINITY;          // the largest and the second largest of the group
            for (int e = g * per; e < (g + 1) * per; ++e) {
                const float v = choice_s[e];
                if (v > a) { b = a; a = v; }
                else if (v > b) b = v;
            }
            rank_s[g] = per > 1 ? a + b : a;
        }
        __syncthreads();
        // the `keep` best groups, one at a time; +infinity in place of its rank marks a kept group
        for (int k = 0; k < keep; ++k) {
            float best = -INFINITY;
            int at = 0x7fffffff;
            for (int g = lane; g < groups; g += kWave) {
                const float v = rank_s[g];
                if (v != INFINITY && (v > best || at == 0x7fffffff)) { best = v; at = g; }
            }
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, kWave);
                const int oa = __shfl_xor(at, off, kWave);
                if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
            }
            if (lane == 0 && at != 0x7fffffff) rank_s[at] = INFINITY;
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i) {
            const int e = lane + kWave * i;
            if (e < E && rank_s[e / per] != INFINITY) c[i] = -INFINITY;
        }
    }
    // the `top` largest choice scores that are left (`gone`: taken already, or no expert at all)
    bool gone[MOE_PER_LANE];
#pragma unroll
    for (int i = 0; i < MOE_PER_LANE; ++i) gone[i] = lane + kWave * i >= E;
    float mine = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i)
            if (!gone[i] && (at == 0x7fffffff || c[i] > best)) { best = c[i]; at = lane + kWave * i; }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, kWave);
            const int oa = __shfl_xor(at, off, kWave);
            if (oa != 0x7fffffff && (at == 0x7fffffff || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
        }
#pragma unroll
        for (int i = 0; i < MOE_PER_LANE; ++i)
            if (lane + kWave * i == at) gone[i] = true;
        if (lane == 0) ids[(size_t)t * top + k] = at;
        if (lane == k) mine = score_s[at] * scale;
    }
    if (lane < top) weights[(size_t)t * top + lane] = mine;
}

// One workgroup: counts, the two running sums, and every pair's sorted row.
__global__ __launch_bounds__(1024) void moe_lists_kernel(const int* __restrict__ ids, int n, int top, int E,
                                                         int tile, int* __restrict__ row_start,
                                                         int* __restrict__ tile_start,
                                                         int* __restrict__ sorted_token,
                                                         int* __restrict__ entry_row) {
    __shared__ int counts[MOE_MAX_EXPERTS];
    __shared__ int cursor[MOE_MAX_EXPERTS];
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) counts[e] = 0;
    __syncthreads();
    for (int i = tid; i < n; i += blockDim.x) atomicAdd(&counts[ids[i]], 1);
    __syncthreads();
    if (tid == 0) {
        int rows = 0, tiles = 0;
        for (int e = 0; e < E; ++e) {
            row_start[e] = rows;
            tile_start[e] = tiles;
            cursor[e] = rows;
            rows += counts[e];
            tiles += (counts[e] + tile - 1) / tile;
        }
        row_start[E] = rows;
        tile_start[E] = tiles;
    }
    __syncthreads();
    for (int i = tid; i < n; i += blockDim.x) {
        const int row = atomicAdd(&cursor[ids[i]], 1);
        sorted_token[row] = i / top;
        entry_row[i] = row;
    }
}

template <typename T>
__global__ void moe_combine_kernel(const float* __restrict__ y, const float* __restrict__ weights,
                                   const int* __restrict__ entry_row, int top, int n, T* __restrict__ out) {
    const int t = blockIdx.x;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float total = 0.f;
        for (int k = 0; k < top; ++k)
            total = fmaf(weights[(size_t)t * top + k], y[(size_t)entry_row[(size_t)t * top + k] * n + i], total);
        out[(size_t)t * n + i] = from_f32<T>(total);
    }
}

// the same plus sigmoid(gates[t, gate_column]) * shared[t]; weights null: every choice counts 1; gates null: the
// shared rows count 1
template <typename T, typename TS>
__global__ void moe_combine_shared_kernel(const float* __restrict__ y, const float* __restrict__ weights,
                                          const int* __restrict__ entry_row, int top, int n,
                                          const TS* __restrict__ shared, const float* __restrict__ gates, int gate_cols,
                                          int gate_column, T* __restrict__ out) {
    const int t = blockIdx.x;
    const float g = gates ? 1.f / (1.f + expf(-gates[(size_t)t * gate_cols + gate_column])) : 1.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float total = 0.f;
        for (int k = 0; k < top; ++k)
            total = fmaf(weights ? weights[(size_t)t * top + k] : 1.f, y[(size_t)entry_row[(size_t)t * top + k] * n + i], total);
        out[(size_t)t * n + i] = from_f32<T>(shared ? fmaf(g, to_f32(shared[(size_t)t * n + i]), total) : total);
    }
}

// Sorted row entry_row[e] of entry e (a token's choice): act(w gate) * (w up) with w = weights[e], which is what
// the gated expert makes of w times its input (both products are linear).  gu [rows, 2 I] -> out [rows, I]
template <typename T>
__global__ void gated_activation_weighted_kernel(const T* __restrict__ gu, T* __restrict__ out,
                                                 const float* __restrict__ weights, const int* __restrict__ entry_row,
                                                 int I, int kind, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t e = idx / I, i = idx % I;
        const size_t row = (size_t)entry_row[e];
        const float w = weights[e];
        const float g = w * to_f32(gu[row * 2 * I + i]), u = w * to_f32(gu[row * 2 * I + I + i]);
        out[row * I + i] = from_f32<T>((kind == 0 ? g * sigmoid(g) : activate(g, ACT_GELU_TANH)) * u);
    }
}

}  // namespace lc

using namespace lc;

// gu [entries, 2 I] (sorted rows) -> out [entries, I]; weights float32 [entries], entry_row int32 [entries];
// kind 0: silu, 1: gelu (tanh form)
LC_API int lc_gated_activation_weighted(const void* gu, void* out, int dt, const float* weights, const int* entry_row,
                                        int entries, int I, int kind, hipStream_t stream) {
    LC_CHECK(entries >= 0 && I > 0 && (kind == 0 || kind == 1), "gated_activation_weighted: bad arguments");
    if (entries == 0) return 0;
    LC_CHECK(gu && out && weights && entry_row, "gated_activation_weighted: null pointer");
    const size_t total = (size_t)entries * I;
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    if (dt == DT_F32)
        gated_activation_weighted_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, weights,
                                                                            entry_row, I, kind, total);
    else if (dt == DT_BF16)
        gated_activation_weighted_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, weights, entry_row,
                                                                           I, kind, total);
    else
        LC_CHECK(false, "gated_activation_weighted: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("gated_activation_weighted");
    return 0;
}

LC_API int lc_moe_max_experts(void) { return MOE_MAX_EXPERTS; }

// logits float32 [T, E] -> ids int32 [T, top], weights float32 [T, top]
LC_API int lc_moe_route(const float* logits, int T, int E, int top, int renormalise, float eps, int* ids,
                        float* weights, hipStream_t stream) {
    LC_CHECK(T >= 0 && E > 0 && top > 0 && top <= E, "moe route: bad sizes T=%d E=%d top=%d", T, E, top);
    LC_CHECK(E <= MOE_MAX_EXPERTS, "moe route: %d experts are above the supported %d", E, MOE_MAX_EXPERTS);
    LC_CHECK(top <= kWave, "moe route: %d choices a token are above the supported %d", top, kWave);
    if (T == 0) return 0;
    LC_CHECK(logits && ids && weights, "moe route: null pointer");
    moe_route_kernel<<<T, kWave, 0, stream>>>(logits, E, top, renormalise, eps, ids, weights);
    LC_LAUNCH_CHECK("moe_route");
    return 0;
}

// ids [T * top] -> row_start, tile_start [E + 1], sorted_token [T * top], entry_row [T * top]
LC_API int lc_moe_lists(const int* ids, int T, int top, int E, int tile, int* row_start, int* tile_start,
                        int* sorted_token, int* entry_row, hipStream_t stream) {
    LC_CHECK(T >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && tile > 0, "moe lists: bad sizes");
    LC_CHECK(ids && row_start && tile_start && sorted_token && entry_row, "moe lists: null pointer");
    LC_CHECK((long long)T * top < (1ll << 31), "moe lists: too many rows");
    moe_lists_kernel<<<1, 1024, 0, stream>>>(ids, T * top, top, E, tile, row_start, tile_start, sorted_token, entry_row);
    LC_LAUNCH_CHECK("moe_lists");
    return 0;
}

// y float32 [T * top, n] -> out [T, n]
LC_API int lc_moe_combine(const float* y, const float* weights, const int* entry_row, int T, int top, int n,
                          void* out, int dt, hipStream_t stream) {
    LC_CHECK(T >= 0 && top > 0 && n > 0, "moe combine: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(y && weights && entry_row && out, "moe combine: null pointer");
    const int threads = n >= 1024 ? 256 : (n >= 256 ? 128 : 64);
    if (dt == DT_F32)
        moe_combine_kernel<float><<<T, threads, 0, stream>>>(y, weights, entry_row, top, n, (float*)out);
    else if (dt == DT_BF16)
        moe_combine_kernel<bf16><<<T, threads, 0, stream>>>(y, weights, entry_row, top, n, (bf16*)out);
    else
        LC_CHECK(false, "moe combine: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("moe_combine");
    return 0;
}

// logits float32 [T, cols] (the experts' in the first E columns), bias [E] or null -> ids, weights [T, top]
LC_API int lc_moe_route_logits(const float* logits, int cols, const float* bias, int T, int E, int top, int* ids,
                               float* weights, hipStream_t stream) {
    LC_CHECK(T >= 0 && E > 0 && top > 0 && top <= E && cols >= E, "moe route: bad sizes T=%d E=%d top=%d cols=%d", T, E,
             top, cols);
    LC_CHECK(E <= MOE_MAX_EXPERTS, "moe route: %d experts are above the supported %d", E, MOE_MAX_EXPERTS);
    LC_CHECK(top <= kWave, "moe route: %d choices a token are above the supported %d", top, kWave);
    if (T == 0) return 0;
    LC_CHECK(logits && ids && weights, "moe route: null pointer");
    moe_route_logits_kernel<<<T, kWave, 0, stream>>>(logits, cols, bias, E, top, ids, weights);
    LC_LAUNCH_CHECK("moe_route_logits");
    return 0;
}

// y float32 [T * top, n], shared [T, n], gates float32 [T, gate_cols] -> out [T, n]
LC_API int lc_moe_combine_shared(const float* y, const float* weights, const int* entry_row, int T, int top, int n,
                                 const void* shared, int dt_shared, const float* gates, int gate_cols, int gate_column,
                                 void* out, int dt, hipStream_t stream) {
    LC_CHECK(T >= 0 && top > 0 && n > 0 && (!gates || (gate_cols > 0 && gate_column >= 0 && gate_column < gate_cols)),
             "moe combine: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(y && entry_row && out && (shared || !gates), "moe combine: null pointer");
    const int threads = n >= 1024 ? 256 : (n >= 256 ? 128 : 64);
#define LC_COMBINE(TO, TS)                                                                                       \
    moe_combine_shared_kernel<TO, TS><<<T, threads, 0, stream>>>(y, weights, entry_row, top, n, (const TS*)shared, \
                                                                 gates, gate_cols, gate_column, (TO*)out)
    if (dt == DT_F32 && dt_shared == DT_F32) LC_COMBINE(float, float);
    else if (dt == DT_F32 && dt_shared == DT_BF16) LC_COMBINE(float, bf16);
    else if (dt == DT_BF16 && dt_shared == DT_F32) LC_COMBINE(bf16, float);
    else if (dt == DT_BF16 && dt_shared == DT_BF16) LC_COMBINE(bf16, bf16);
    else LC_CHECK(false, "moe combine: unknown dtypes %d, %d", dt, dt_shared);
#undef LC_COMBINE
    LC_LAUNCH_CHECK("moe_combine_shared");
    return 0;
}

// logits float32 [T, E], correction float32 [E] or null -> ids int32 [T, top], weights float32 [T, top]
LC_API int lc_moe_route_sigmoid(const float* logits, const float* correction, int T, int E, int top, int groups,
                                int keep, float scale, int* ids, float* weights, hipStream_t stream) {
    LC_CHECK(T >= 0 && E > 0 && E <= MOE_MAX_EXPERTS && top > 0 && top <= kWave, "moe route: bad sizes E=%d top=%d", E, top);
    LC_CHECK(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (E / groups),
             "moe route: %d groups of which %d are kept do not hold %d choices among %d experts", groups, keep, top, E);
    if (T == 0) return 0;
    LC_CHECK(logits && ids && weights, "moe route: null pointer");
    moe_route_sigmoid_kernel<<<T, kWave, 0, stream>>>(logits, correction, E, top, groups, keep, scale, ids, weights);
    LC_LAUNCH_CHECK("moe_route_sigmoid");
    return 0;
}
