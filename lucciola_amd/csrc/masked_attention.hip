// Attention over a paged cache with the things the framework's other attention kernels do not know:
// keys and values of different head counts and sizes, several score maps per head over the same values
// (differential attention), a mask of chunks, a bias that grows with the logarithm of the distance, and a
// sink in the softmax's denominator.  Float32 arithmetic throughout; one workgroup per token and head.
//
// With p the query's position, the visible keys are lo .. p, lo = max(p - p % chunk (chunk > 0),
// p - window + 1 (window > 0), 0).  Per head h (kv head g = h / (heads / kv_heads)) and map m < maps:
//   s_j = scale (q_(h,m) . k_(g,m),j) - r1_h ln(1 + r2_h (p - j))            (the bias where r1 is given)
//   a_m = sum_j exp(s_j) v_g,j / (sum_j exp(s_j) + exp(sink_h))              (the sink where it is given)
//   maps = 1: o = a_0;   maps = 2: o = a_0 - lambda a_1
//   unit_out: o <- o / sqrt(mean(o^2) + eps) * out_scale;   gate: o <- o sigmoid(gate_(h, .))
// Cache layouts: keys token-major, [pages, page, kv_heads * maps * d]; values transposed inside a page, [pages,
// kv_heads * dv, page] (the matrix-core kernel's operand wants a value entry's neighbouring keys side by side).
// Position j of request r lies in page block_table[r][j / page] at place j % page.
//
// The keys are walked in tiles of 256 from lo on, with a running maximum and sum per map: the order of
// every addition is a function of the query's position alone, so a token's result has the same bits in
// every batch and for every cut of its prompt.
//
// This file also holds the prologue that makes q, k and v of a step from the float32 projections: an
// optional short convolution over time per channel, an optional rotation of neighbouring pairs
// (entries 2i, 2i + 1 of the first `rot` entries of every q and k head), an optional division of every q
// and k head by its root mean square; q goes to a tensor, k and v into their cache rows.
#include "common.h"
#include "short_conv.h"

namespace lc {

constexpr int MA_THREADS = 256;
constexpr int MA_MAX = 256;          // entries of a query/key head and of a value head at most
constexpr int MA_MAPS = 2;           // score maps a head at most

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ krow, int d) {
    float dot = 0.f;
    if ((d & 3) == 0) {
        for (int e = 0; e < d; e += 4) {
            float k4[4];
            load4(k4, krow + e);
            dot = fmaf(qs[e], k4[0], dot);
            dot = fmaf(qs[e + 1], k4[1], dot);
            dot = fmaf(qs[e + 2], k4[2], dot);
            dot = fmaf(qs[e + 3], k4[3], dot);
        }
    } else {
        for (int e = 0; e < d; ++e) dot = fmaf(qs[e], to_f32(krow[e]), dot);
    }
    return dot;
}

template <typename T, int MAPS>
__global__ __launch_bounds__(MA_THREADS) void masked_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ tok_req, const int* __restrict__ positions, const int* __restrict__ block_table,
    int max_blocks, int page_size, int heads, int kv_heads, int d, int dv, int dv_pow2, float scale, int chunk,
    int window, const float* __restrict__ r1, const float* __restrict__ r2, const float* __restrict__ sink,
    float lambda, int unit_out, float eps, float out_scale, const float* __restrict__ gate, int gate_stride,
    int gate_column, T* __restrict__ out) {
    __shared__ __align__(16) float qs[MAPS][MA_MAX];
    __shared__ float ps[MAPS][MA_THREADS];
    __shared__ float scratch[16];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int g = h / (heads / kv_heads);
    const int r = tok_req[t], p = positions[t];
    int lo = 0;
    if (chunk > 0) lo = p - p % chunk;
    if (window > 0) lo = max(lo, p - window + 1);
    const int* table = block_table + (size_t)r * max_blocks;
    const size_t k_row = (size_t)kv_heads * MAPS * d, v_row = (size_t)kv_heads * dv;
    for (int i = tid; i < MAPS * d; i += MA_THREADS) {
        const int m = i / d, e = i % d;
        qs[m][e] = to_f32(q[((size_t)t * heads + h) * MAPS * d + i]) * scale;
    }
    const float bias1 = r1 ? r1[h] : 0.f, bias2 = r1 ? r2[h] : 0.f;
    const int groups = MA_THREADS / dv_pow2, grp = tid / dv_pow2, dim = tid % dv_pow2;
    const bool active = dim < dv;
    float M[MAPS], L[MAPS], acc[MAPS];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) { M[m] = -INFINITY; L[m] = 0.f; acc[m] = 0.f; }
    __syncthreads();
    for (int c0 = lo; c0 <= p; c0 += MA_THREADS) {
        const int count = min(MA_THREADS, p - c0 + 1);
        float s[MAPS];
#pragma unroll
        for (int m = 0; m < MAPS; ++m) s[m] = -INFINITY;
        if (tid < count) {
            const int j = c0 + tid;
            const size_t row = (size_t)table[j / page_size] * page_size + j % page_size;
            const float far = r1 ? bias1 * log1pf(bias2 * (float)(p - j)) : 0.f;
#pragma unroll
            for (int m = 0; m < MAPS; ++m)
                s[m] = dot_row(qs[m], k_cache + row * k_row + ((size_t)g * MAPS + m) * d, d) - far;
        }
#pragma unroll
        for (int m = 0; m < MAPS; ++m) {
            const float m_new = fmaxf(M[m], block_max(s[m], scratch));
            const float alpha = expf(M[m] - m_new);          // 0 on the first tile (M = -inf)
            const float pj = tid < count ? expf(s[m] - m_new) : 0.f;
            ps[m][tid] = pj;
            L[m] = fmaf(L[m], alpha, block_sum(pj, scratch));
            acc[m] *= alpha;
            M[m] = m_new;
        }
        __syncthreads();
        if (active)
            for (int jj = grp; jj < count; jj += groups) {
                const int j = c0 + jj;
                const float v = to_f32(v_cache[((size_t)table[j / page_size] * v_row + (size_t)g * dv + dim) * page_size
                                               + j % page_size]);
#pragma unroll
                for (int m = 0; m < MAPS; ++m) acc[m] = fmaf(ps[m][jj], v, acc[m]);
            }
        __syncthreads();          // ps is written again by the next tile
    }
    // the key groups' sums of a dim, added from group 0 on; ps is free now
    float a[MAPS];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
        ps[m][tid] = acc[m];
        __syncthreads();
        float total = 0.f;
        if (tid < dv)
            for (int gg = 0; gg < groups; ++gg) total += ps[m][gg * dv_pow2 + tid];
        // the sink: one more term exp(sink) in the denominator, at the joint maximum
        float top = M[m], sunk = 0.f;
        if (sink) {
            top = fmaxf(M[m], sink[h]);
            sunk = expf(sink[h] - top);
        }
        const float shrink = expf(M[m] - top);
        a[m] = total * shrink / fmaf(L[m], shrink, sunk);
    }
    float o = a[0];
    if constexpr (MAPS == 2) o = fmaf(-lambda, a[1], a[0]);
    if (unit_out) {
        const float ss = block_sum(tid < dv ? o * o : 0.f, scratch);
        o = o / sqrtf(ss / (float)dv + eps) * out_scale;
    }
    if (tid < dv) {
        if (gate) o = o / (1.f + expf(-gate[(size_t)t * gate_stride + gate_column + (size_t)h * dv + tid]));
        out[((size_t)t * heads + h) * dv + tid] = from_f32<T>(o);
    }
}

// One wave per (token, head of q | k | v).  proj float32 [T, cols], its first columns: q (nq heads of d) | k (nk of
// d) | v (nv of dv).  taps [C, K] and tails [slots, K - 1, C] with C = all of these columns, or null.
// table float32 [positions, rot] (cosines, then sines of the rot / 2 angles) or null.
template <typename T>
__global__ __launch_bounds__(MA_THREADS) void attention_prepare_kernel(
    const float* __restrict__ proj, int cols, int T_, int nq, int nk, int nv, int d, int dv,
    const float* __restrict__ taps, int K, const float* __restrict__ tails, const int* __restrict__ tok_req,
    const int* __restrict__ q_offsets, const int* __restrict__ slot_ids, const float* __restrict__ table, int rot,
    const int* __restrict__ positions, int unit, float eps, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int* __restrict__ rows, int page_size) {
    const int t = blockIdx.x, lane = threadIdx.x & (kWave - 1);
    const int u = blockIdx.y * (MA_THREADS / kWave) + threadIdx.x / kWave;
    if (u >= nq + nk + nv) return;
    const bool is_v = u >= nq + nk;
    const int width = is_v ? dv : d;
    const int col0 = u < nq ? u * d : (u < nq + nk ? nq * d + (u - nq) * d : (nq + nk) * d + (u - nq - nk) * dv);
    const int C = (nq + nk) * d + nv * dv;
    int local = 0;
    const float* tail = nullptr;
    if (taps) {
        const int r = tok_req[t];
        local = t - q_offsets[r];
        tail = tails + (size_t)slot_ids[r] * (K - 1) * C;
    }
    // a lane holds the pairs lane, lane + 64 of the head: entries 2i and 2i + 1
    float x[2][2], ss = 0.f;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int i = lane + kWave * k;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int at = 2 * i + e;
            x[k][e] = 0.f;
            if (at < width)
                x[k][e] = taps ? short_conv(proj, cols, t, local, col0 + at, taps, K, tail, C)
                               : proj[(size_t)t * cols + col0 + at];
        }
        if (table && !is_v && 2 * i + 1 < rot) {
            const float* angle = table + (size_t)positions[t] * rot;
            const float c = angle[i], s = angle[rot / 2 + i];
            const float a = x[k][0], b = x[k][1];
            x[k][0] = a * c - b * s;
            x[k][1] = fmaf(b, c, a * s);
        }
        ss = fmaf(x[k][0], x[k][0], ss);
        ss = fmaf(x[k][1], x[k][1], ss);
    }
    float inv = 1.f;
    if (unit && !is_v) inv = 1.f / sqrtf(wave_sum(ss) / (float)width + eps);
    T* dst;
    size_t step = 1;                // between neighbouring entries of the head
    if (u < nq) {
        dst = q_out + (size_t)t * nq * d + (size_t)u * d;
    } else {
        if (!rows || rows[t] < 0) return;
        if (is_v) {                 // values lie transposed inside their page: [entry][place]
            dst = v_cache + ((size_t)(rows[t] / page_size) * nv * dv + (size_t)(u - nq - nk) * dv) * page_size
                  + rows[t] % page_size;
            step = page_size;
        } else {
            dst = k_cache + (size_t)rows[t] * nk * d + (size_t)(u - nq) * d;
        }
    }
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int at = 2 * (lane + kWave * k) + e;
            if (at < width) dst[at * step] = from_f32<T>(x[k][e] * inv);
        }
}

// The same for steps without the unit norm, where nothing is summed over a head: a thread per pair of neighbouring
// entries of the whole row (head sizes and the row's stride even), the pair's inputs and taps in wide loads.  The sums
// and the rotation are written as in the kernel above, so both give the same bits.
template <typename T>
__global__ void attention_prepare_pairs_kernel(
    const float* __restrict__ proj, int cols, int T_, int nq, int nk, int nv, int d, int dv,
    const float* __restrict__ taps, int K, const float* __restrict__ tails, const int* __restrict__ tok_req,
    const int* __restrict__ q_offsets, const int* __restrict__ slot_ids, const float* __restrict__ table, int rot,
    const int* __restrict__ positions, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ rows, int page_size) {
    const int C = (nq + nk) * d + nv * dv, pairs = C / 2, q_cols = nq * d, qk_cols = (nq + nk) * d;
    const size_t total = (size_t)T_ * pairs;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int t = (int)(idx / pairs), c = 2 * (int)(idx % pairs);
        const bool is_v = c >= qk_cols;
        const int at = is_v ? (c - qk_cols) % dv : c % d;          // the pair's place in its head
        float a, b;
        if (taps) {
            const int r = tok_req[t];
            const int local = t - q_offsets[r];
            const float* tail = tails + (size_t)slot_ids[r] * (K - 1) * C;
            a = b = 0.f;
            for (int back = K - 1; back >= 0; --back) {         // oldest input first
                const float2 in = *reinterpret_cast<const float2*>(
                    back <= local ? proj + (size_t)(t - back) * cols + c : tail + (size_t)((K - 1) - (back - local)) * C + c);
                a = fmaf(taps[(size_t)c * K + (K - 1 - back)], in.x, a);
                b = fmaf(taps[(size_t)(c + 1) * K + (K - 1 - back)], in.y, b);
            }
        } else {
            const float2 in = *reinterpret_cast<const float2*>(proj + (size_t)t * cols + c);
            a = in.x;
            b = in.y;
        }
        if (table && !is_v && at + 1 < rot) {
            const float* angle = table + (size_t)positions[t] * rot;
            const float cs = angle[at / 2], sn = angle[rot / 2 + at / 2];
            const float a0 = a, b0 = b;
            a = a0 * cs - b0 * sn;
            b = fmaf(b0, cs, a0 * sn);
        }
        if (c < q_cols) {
            q_out[(size_t)t * q_cols + c] = from_f32<T>(a);
            q_out[(size_t)t * q_cols + c + 1] = from_f32<T>(b);
        } else if (rows && rows[t] >= 0) {
            if (is_v) {
                T* dst = v_cache + ((size_t)(rows[t] / page_size) * nv * dv + (c - qk_cols)) * page_size + rows[t] % page_size;
                dst[0] = from_f32<T>(a);
                dst[page_size] = from_f32<T>(b);
            } else {
                T* dst = k_cache + (size_t)rows[t] * nk * d + (c - q_cols);
                dst[0] = from_f32<T>(a);
                dst[1] = from_f32<T>(b);
            }
        }
    }
}

}  // namespace lc

using namespace lc;

LC_API int lc_masked_attention(const void* q, const void* k_cache, const void* v_cache, int dt, const int* tok_req,
                               const int* positions, const int* block_table, int max_blocks, int page_size, int T,
                               int heads, int kv_heads, int maps, int d, int dv, float scale, int chunk, int window,
                               const float* r1, const float* r2, const float* sink, float lambda, int unit_out,
                               float eps, float out_scale, const float* gate, int gate_stride, int gate_column,
                               void* out, hipStream_t stream) {
    LC_CHECK(T >= 0 && heads > 0 && kv_heads > 0 && d > 0 && dv > 0 && page_size > 0 && max_blocks > 0,
             "masked attention: bad sizes T=%d heads=%d kv=%d d=%d dv=%d page=%d blocks=%d", T, heads, kv_heads, d, dv,
             page_size, max_blocks);
    if (T == 0) return 0;
    LC_CHECK(heads % kv_heads == 0, "masked attention: %d heads are not a multiple of %d kv heads", heads, kv_heads);
    LC_CHECK(maps == 1 || maps == 2, "masked attention: %d score maps a head (1 or 2)", maps);
    LC_CHECK(d <= MA_MAX && dv <= MA_MAX, "masked attention: heads of %d/%d entries are above %d", d, dv, MA_MAX);
    LC_CHECK(heads <= 65535, "masked attention: too many heads (%d)", heads);
    LC_CHECK(chunk >= 0 && window >= 0, "masked attention: bad mask");
    LC_CHECK(q && k_cache && v_cache && out && tok_req && positions && block_table, "masked attention: null pointer");
    LC_CHECK((r1 == nullptr) == (r2 == nullptr), "masked attention: the bias needs both of its vectors");
    LC_CHECK(!gate || (gate_column >= 0 && gate_column + heads * dv <= gate_stride), "masked attention: bad gate columns");
    int dv_pow2 = 1;
    while (dv_pow2 < dv) dv_pow2 <<= 1;
    const dim3 grid(T, heads);
#define LC_MA(TT, MAPS)                                                                                              \
    masked_attention_kernel<TT, MAPS><<<grid, MA_THREADS, 0, stream>>>(                                               \
        (const TT*)q, (const TT*)k_cache, (const TT*)v_cache, tok_req, positions, block_table, max_blocks, page_size, \
        heads, kv_heads, d, dv, dv_pow2, scale, chunk, window, r1, r2, sink, lambda, unit_out, eps, out_scale, gate,  \
        gate_stride, gate_column, (TT*)out)
    if (dt == DT_F32) { if (maps == 1) LC_MA(float, 1); else LC_MA(float, 2); }
    else if (dt == DT_BF16) { if (maps == 1) LC_MA(bf16, 1); else LC_MA(bf16, 2); }
    else LC_CHECK(false, "masked attention: unknown dtype %d", dt);
#undef LC_MA
    LC_LAUNCH_CHECK("masked_attention");
    return 0;
}

static thread_local int g_prepare_pairs = 1;

// Tests: whether steps without the unit norm may take the kernel with a thread per pair of entries (for the calling
// thread).  Returns the setting before.
LC_API int lc_attention_prepare_pairs(int on) {
    const int before = g_prepare_pairs;
    if (on >= 0) g_prepare_pairs = on ? 1 : 0;
    return before;
}

LC_API int lc_attention_prepare(const float* proj, int cols, int T, int nq, int nk, int nv, int d, int dv,
                                const float* taps, int K, const float* tails, const int* tok_req,
                                const int* q_offsets, const int* slot_ids, const float* table, int rot,
                                const int* positions, int unit, float eps, void* q_out, void* k_cache, void* v_cache,
                                int dt, const int* rows, int page_size, hipStream_t stream) {
    LC_CHECK(T >= 0 && nq > 0 && nk >= 0 && nv >= 0 && d > 0 && dv > 0 && cols >= (nq + nk) * d + nv * dv,
             "attention prepare: bad sizes");
    LC_CHECK(d <= MA_MAX && dv <= MA_MAX, "attention prepare: heads of %d/%d entries are above %d", d, dv, MA_MAX);
    if (T == 0) return 0;
    LC_CHECK(proj && q_out, "attention prepare: null pointer");
    LC_CHECK(!taps || (K >= 1 && K <= SHORT_CONV_MAX_TAPS && tok_req && q_offsets && slot_ids && (K == 1 || tails)),
             "attention prepare: a convolution needs 1 to %d taps, the tails and the request lists", SHORT_CONV_MAX_TAPS);
    LC_CHECK(!table || (rot > 0 && rot % 2 == 0 && rot <= d && positions), "attention prepare: bad rotation");
    LC_CHECK(!rows || (k_cache && v_cache && page_size > 0), "attention prepare: rows without a cache");
    if (!unit && d % 2 == 0 && dv % 2 == 0 && cols % 2 == 0 && g_prepare_pairs) {
        const size_t total = (size_t)T * (((nq + nk) * d + nv * dv) / 2);
        const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
        if (dt == DT_F32)
            attention_prepare_pairs_kernel<float><<<blocks, 256, 0, stream>>>(
                proj, cols, T, nq, nk, nv, d, dv, taps, K, tails, tok_req, q_offsets, slot_ids, table, rot, positions,
                (float*)q_out, (float*)k_cache, (float*)v_cache, rows, page_size > 0 ? page_size : 1);
        else if (dt == DT_BF16)
            attention_prepare_pairs_kernel<bf16><<<blocks, 256, 0, stream>>>(
                proj, cols, T, nq, nk, nv, d, dv, taps, K, tails, tok_req, q_offsets, slot_ids, table, rot, positions,
                (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, rows, page_size > 0 ? page_size : 1);
        else
            LC_CHECK(false, "attention prepare: unknown dtype %d", dt);
        LC_LAUNCH_CHECK("attention_prepare");
        return 0;
    }
    const int units = nq + nk + nv, per = MA_THREADS / kWave;
    const dim3 grid(T, (units + per - 1) / per);
    if (dt == DT_F32)
        attention_prepare_kernel<float><<<grid, MA_THREADS, 0, stream>>>(
            proj, cols, T, nq, nk, nv, d, dv, taps, K, tails, tok_req, q_offsets, slot_ids, table, rot, positions, unit,
            eps, (float*)q_out, (float*)k_cache, (float*)v_cache, rows, page_size);
    else if (dt == DT_BF16)
        attention_prepare_kernel<bf16><<<grid, MA_THREADS, 0, stream>>>(
            proj, cols, T, nq, nk, nv, d, dv, taps, K, tails, tok_req, q_offsets, slot_ids, table, rot, positions, unit,
            eps, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, rows, page_size);
    else
        LC_CHECK(false, "attention prepare: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("attention_prepare");
    return 0;
}
