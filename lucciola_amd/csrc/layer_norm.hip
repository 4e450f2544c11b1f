// Row-wise kernels of layers that norm with mean and variance, add a position vector to the
// embedding, gate one half of a product with the other, and keep attention heads in slots.
// All arithmetic is float32; only loads and stores have the tensors' types.
//   layer norm      y = (v - mean) / sqrt(var + eps) w + b,  var = mean((v - mean)^2)
//   with a stream   v = h + d, where d is the branch output, itself layer-normed first if it
//                   brings weights of its own; h becomes v where asked
//   position vector entry 2i: sin(p f_i), entry 2i + 1: cos(p f_i)
//   gated           act(gate) * up, act = silu or gelu (tanh form)
//   heads in slots  q, k heads divided by their root mean square over their own entries, times a
//                   weight, q also times a factor per head; q, k, v written as heads of `slot`
//                   entries with zeros behind theirs (k, v into the paged cache)
//   head gate norm  every head of a float32 row divided by its root mean square, times a weight,
//                   times sigmoid or silu of a gate
#include "common.h"

#include "activations.h"

namespace lc {

__device__ __forceinline__ float silu(float z) { return z / (1.f + expf(-z)); }

// Mean and inverse deviation of the n floats in `row` (LDS); every thread gets both.
__device__ __forceinline__ void row_moments(const float* row, int n, float eps, float* scratch, float& mean,
                                            float& inv) {
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) s += row[i];
    mean = block_sum(s, scratch) / (float)n;
    float q = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const float d = row[i] - mean;
        q = fmaf(d, d, q);
    }
    inv = 1.f / sqrtf(block_sum(q, scratch) / (float)n + eps);
}

// One workgroup per output row r; src row = rows ? rows[r] : r.
//   d = delta[src], layer-normed with (pw, pb, peps) if pw;  v = h ? h[src] + dscale d : d
//   if (write_h) h[src] = v;  out[r] = w ? layer norm of v with (w, b, eps) : v
template <typename TD, typename TO>
__global__ void layer_norm_kernel(float* __restrict__ h, const TD* __restrict__ delta, float dscale,
                                  const float* __restrict__ pw,
                                  const float* __restrict__ pb, float peps, const int* __restrict__ rows,
                                  const float* __restrict__ w, const float* __restrict__ b, float eps,
                                  TO* __restrict__ out, int n, int write_h) {
    extern __shared__ float row[];
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? rows[r] : r;
    float mean, inv;
    if (delta) {
        const TD* dr = delta + src * n;
        for (int i = threadIdx.x; i < n; i += blockDim.x) row[i] = to_f32(dr[i]);
        if (pw) {
            __syncthreads();
            row_moments(row, n, peps, scratch, mean, inv);
            for (int i = threadIdx.x; i < n; i += blockDim.x) row[i] = fmaf((row[i] - mean) * inv, pw[i], pb[i]);
        }
    }
    if (h) {
        float* hr = h + src * n;
        for (int i = threadIdx.x; i < n; i += blockDim.x) {     // a thread meets its own entries only
            const float v = delta ? fmaf(dscale, row[i], hr[i]) : hr[i];
            row[i] = v;
            if (write_h) hr[i] = v;
        }
    }
    __syncthreads();
    TO* o = out + (size_t)r * n;
    if (!w) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) o[i] = from_f32<TO>(row[i]);
        return;
    }
    row_moments(row, n, eps, scratch, mean, inv);
    for (int i = threadIdx.x; i < n; i += blockDim.x) o[i] = from_f32<TO>(fmaf((row[i] - mean) * inv, w[i], b[i]));
}

// The same for rows of up to ITEMS entries a thread: every operand is asked for before the first
// sum, so a row costs one trip to memory and not one per stage.
template <typename TD, typename TO, int ITEMS>
__global__ void layer_norm_rows_kernel(float* __restrict__ h, const TD* __restrict__ delta, float dscale,
                                       const float* __restrict__ pw, const float* __restrict__ pb, float peps,
                                       const int* __restrict__ rows, const float* __restrict__ w,
                                       const float* __restrict__ b, float eps, TO* __restrict__ out, int n,
                                       int write_h) {
    __shared__ float scratch[16];
    const int r = blockIdx.x, tid = threadIdx.x, step = blockDim.x;
    const size_t src = rows ? rows[r] : r;
    float d[ITEMS], hv[ITEMS], wv[ITEMS], bv[ITEMS], pwv[ITEMS], pbv[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int i = tid + k * step;
        const bool ok = i < n;
        d[k] = (delta && ok) ? to_f32(delta[src * n + i]) : 0.f;
        hv[k] = (h && ok) ? h[src * n + i] : 0.f;
        wv[k] = (w && ok) ? w[i] : 0.f;
        bv[k] = (w && ok) ? b[i] : 0.f;
        pwv[k] = (pw && ok) ? pw[i] : 0.f;
        pbv[k] = (pw && ok) ? pb[i] : 0.f;
    }
    const float inv_n = 1.f / (float)n;
    if (delta && pw) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) s += d[k];
        const float mean = block_sum(s, scratch) * inv_n;
        float q = 0.f;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            d[k] = tid + k * step < n ? d[k] - mean : 0.f;
            q = fmaf(d[k], d[k], q);
        }
        const float inv = 1.f / sqrtf(block_sum(q, scratch) * inv_n + peps);
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) d[k] = fmaf(d[k] * inv, pwv[k], pbv[k]);
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int i = tid + k * step;
        const float v = h ? (delta ? fmaf(dscale, d[k], hv[k]) : hv[k]) : d[k];
        d[k] = i < n ? v : 0.f;
        if (h && delta && write_h && i < n) h[src * n + i] = v;
        s += d[k];
    }
    TO* o = out + (size_t)r * n;
    if (!w) {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            if (tid + k * step < n) o[tid + k * step] = from_f32<TO>(d[k]);
        return;
    }
    const float mean = block_sum(s, scratch) * inv_n;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        d[k] = tid + k * step < n ? d[k] - mean : 0.f;
        q = fmaf(d[k], d[k], q);
    }
    const float inv = 1.f / sqrtf(block_sum(q, scratch) * inv_n + eps);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
        if (tid + k * step < n) o[tid + k * step] = from_f32<TO>(fmaf(d[k] * inv, wv[k], bv[k]));
}

// A thread per pair of entries: one angle, its sine and its cosine.
template <typename T>
__global__ void embedding_sinusoid_kernel(const int* __restrict__ ids, const int* __restrict__ positions,
                                          const T* __restrict__ table, const float* __restrict__ freq,
                                          float* __restrict__ out, int H, int V, float scale) {
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= V ? V - 1 : id);
    const float p = (float)positions[t];
    const T* rowp = table + (size_t)id * H;
    for (int pair = threadIdx.x; 2 * pair < H; pair += blockDim.x) {
        float sn, cs;
        sincosf(p * freq[pair], &sn, &cs);
        const int i = 2 * pair;
        out[(size_t)t * H + i] = fmaf(to_f32(rowp[i]), scale, sn);
        if (i + 1 < H) out[(size_t)t * H + i + 1] = fmaf(to_f32(rowp[i + 1]), scale, cs);
    }
}

template <typename T>
__global__ void gated_activation_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, int kind, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const size_t t = idx / I, i = idx % I;
        const float g = to_f32(gu[t * 2 * I + i]), u = to_f32(gu[t * 2 * I + I + i]);
        out[idx] = from_f32<T>((kind == 0 ? silu(g) : activate(g, ACT_GELU_TANH)) * u);
    }
}

constexpr int HEAD_MAX = 256;                  // entries of a head at most: four a lane
constexpr int HEAD_PER_LANE = HEAD_MAX / kWave;

// One wave per (token, head of q | k | v).
template <typename T>
__global__ __launch_bounds__(kWave) void head_norm_write_kernel(
    const T* __restrict__ proj, int nh, int nkv, int d, int dv, int slot, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const float* __restrict__ head_scale, T* __restrict__ q_out,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ slots, int page_size, int num_pages) {
    const int per_token = nh + 2 * nkv;
    const int t = blockIdx.x / per_token, which = blockIdx.x % per_token, lane = threadIdx.x;
    const size_t cols = (size_t)nh * d + (size_t)nkv * (d + dv);
    const T* row = proj + (size_t)t * cols;
    if (which < nh + nkv) {                    // a q or k head: norm over its d entries
        const bool is_q = which < nh;
        const int head = is_q ? which : which - nh;
        const T* x = row + (is_q ? (size_t)head * d : (size_t)nh * d + (size_t)head * d);
        const float* w = is_q ? qw : kw;
        float v[HEAD_PER_LANE], ss = 0.f;
#pragma unroll
        for (int j = 0; j < HEAD_PER_LANE; ++j) {
            const int i = lane + kWave * j;
            v[j] = i < d ? to_f32(x[i]) : 0.f;
            ss = fmaf(v[j], v[j], ss);
        }
        float factor = 1.f;
        if (w) factor = 1.f / sqrtf(wave_sum(ss) / (float)d + eps);
        const float extra = (is_q && head_scale) ? head_scale[head] : 1.f;
        T* dst;
        if (is_q) {
            dst = q_out + ((size_t)t * nh + head) * slot;
        } else {
            const int s = slots ? slots[t] : -1;
            if (s < 0 || !k_cache || s / page_size >= num_pages) return;
            dst = k_cache + (((size_t)(s / page_size) * nkv + head) * page_size + s % page_size) * slot;
        }
#pragma unroll
        for (int j = 0; j < HEAD_PER_LANE; ++j) {
            const int i = lane + kWave * j;
            if (i < slot) dst[i] = from_f32<T>(i < d ? (w ? v[j] * factor * w[i] : v[j]) * extra : 0.f);
        }
        return;
    }
    const int head = which - nh - nkv;         // a v head: into its page, transposed
    const int s = slots ? slots[t] : -1;
    if (s < 0 || !v_cache || s / page_size >= num_pages) return;
    const T* x = row + (size_t)(nh + nkv) * d + (size_t)head * dv;
    T* dst = v_cache + ((size_t)(s / page_size) * nkv + head) * slot * page_size + s % page_size;
    for (int i = lane; i < slot; i += kWave) dst[(size_t)i * page_size] = i < dv ? x[i] : from_f32<T>(0.f);
}

// One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(kWave) void head_gate_norm_kernel(const float* __restrict__ o,
                                                               const float* __restrict__ gates, int gate_cols,
                                                               int gate_column, const float* __restrict__ weight,
                                                               int per_head, float eps, int gate, int heads, int dim,
                                                               T* __restrict__ out) {
    const int t = blockIdx.x / heads, head = blockIdx.x % heads, lane = threadIdx.x;
    const float* x = o + ((size_t)t * heads + head) * dim;
    const float* g = gates + (size_t)t * gate_cols + gate_column + (size_t)head * dim;
    const float* w = weight + (per_head ? (size_t)head * dim : 0);
    float ss = 0.f;
    for (int i = lane; i < dim; i += kWave) ss = fmaf(x[i], x[i], ss);
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)dim + eps);
    T* dst = out + ((size_t)t * heads + head) * dim;
    for (int i = lane; i < dim; i += kWave) {
        const float z = g[i];
        dst[i] = from_f32<T>(x[i] * inv * w[i] * (gate == 0 ? sigmoid(z) : silu(z)));
    }
}

static int blocks_for(size_t total) { return (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192); }

}  // namespace lc

using namespace lc;

// h float32 [T, n] or null; delta [T, n] of dtype dt_delta or null; (pw, pb, peps): the branch's own
// norm or null; rows int32 [R] or null; (w, b, eps): the norm of the sum, or null to leave it as it is
LC_API int lc_layer_norm(float* h, const void* delta, int dt_delta, float dscale, const float* pw, const float* pb, float peps,
                         const int* rows, const float* w, const float* b, float eps, void* out, int dt_out, int R,
                         int n, int write_h, int T, hipStream_t stream) {
    LC_CHECK(R >= 0 && n > 0 && T >= 0, "layer_norm: bad sizes R=%d n=%d", R, n);
    if (R == 0) return 0;
    LC_CHECK((h || delta) && out, "layer_norm: null pointer");
    LC_CHECK((w == nullptr) == (b == nullptr) && (pw == nullptr) == (pb == nullptr), "layer_norm: a weight without its bias");
    LC_CHECK(!(rows && write_h), "layer_norm: gathered rows cannot be written back");
    LC_CHECK(!pw || delta, "layer_norm: a branch norm without a branch");
    LC_CHECK(n <= 16384, "layer_norm: rows of %d entries are above the kernel's 16384", n);
    constexpr int ITEMS = 8;
    const bool in_registers = n <= ITEMS * 1024;
    const int threads = in_registers ? (((n + ITEMS - 1) / ITEMS + kWave - 1) / kWave) * kWave
                                     : (n >= 1024 ? 256 : (n >= 256 ? 128 : 64));
    const size_t lds = (size_t)n * sizeof(float);
#define LC_LN(TD, TO)                                                                                           \
    if (in_registers)                                                                                           \
        layer_norm_rows_kernel<TD, TO, ITEMS><<<R, threads, 0, stream>>>(h, (const TD*)delta, dscale, pw, pb, peps, rows, w, \
                                                                         b, eps, (TO*)out, n, write_h);         \
    else                                                                                                        \
        layer_norm_kernel<TD, TO><<<R, threads, lds, stream>>>(h, (const TD*)delta, dscale, pw, pb, peps, rows, w, b, eps, \
                                                               (TO*)out, n, write_h)
    const int dd = delta ? dt_delta : DT_F32;
    if (dd == DT_F32 && dt_out == DT_F32) LC_LN(float, float);
    else if (dd == DT_F32 && dt_out == DT_BF16) LC_LN(float, bf16);
    else if (dd == DT_BF16 && dt_out == DT_F32) LC_LN(bf16, float);
    else if (dd == DT_BF16 && dt_out == DT_BF16) LC_LN(bf16, bf16);
    else LC_CHECK(false, "layer_norm: unknown dtypes %d, %d", dt_delta, dt_out);
#undef LC_LN
    LC_LAUNCH_CHECK("layer_norm");
    return 0;
}

LC_API int lc_embedding_sinusoid(const int* ids, const int* positions, const void* table, int dt, const float* freq,
                                 float* out, int T, int H, int V, float scale, hipStream_t stream) {
    LC_CHECK(T >= 0 && H > 0 && V > 0, "embedding_sinusoid: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(ids && positions && table && freq && out, "embedding_sinusoid: null pointer");
    const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
    if (dt == DT_F32)
        embedding_sinusoid_kernel<float><<<T, threads, 0, stream>>>(ids, positions, (const float*)table, freq, out, H, V, scale);
    else if (dt == DT_BF16)
        embedding_sinusoid_kernel<bf16><<<T, threads, 0, stream>>>(ids, positions, (const bf16*)table, freq, out, H, V, scale);
    else
        LC_CHECK(false, "embedding_sinusoid: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("embedding_sinusoid");
    return 0;
}

// gu [T, 2 I] -> out [T, I]; kind 0: silu, 1: gelu (tanh form)
LC_API int lc_gated_activation(const void* gu, void* out, int dt, int T, int I, int kind, hipStream_t stream) {
    LC_CHECK(T >= 0 && I > 0 && (kind == 0 || kind == 1), "gated_activation: bad arguments");
    if (T == 0) return 0;
    LC_CHECK(gu && out, "gated_activation: null pointer");
    const size_t total = (size_t)T * I;
    if (dt == DT_F32)
        gated_activation_kernel<float><<<blocks_for(total), 256, 0, stream>>>((const float*)gu, (float*)out, I, kind, total);
    else if (dt == DT_BF16)
        gated_activation_kernel<bf16><<<blocks_for(total), 256, 0, stream>>>((const bf16*)gu, (bf16*)out, I, kind, total);
    else
        LC_CHECK(false, "gated_activation: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("gated_activation");
    return 0;
}

LC_API int lc_head_norm_write(const void* proj, int dt, int T, int nh, int nkv, int d, int dv, int slot,
                              const float* qw, const float* kw, float eps, const float* head_scale, void* q_out,
                              void* k_cache, void* v_cache, const int* slots, int page_size, int num_pages,
                              hipStream_t stream) {
    LC_CHECK(T >= 0 && nh > 0 && nkv >= 0 && d > 0 && dv > 0, "head_norm_write: bad sizes");
    LC_CHECK(d <= slot && dv <= slot && slot <= HEAD_MAX, "head_norm_write: heads of %d/%d in slots of %d (at most %d)",
             d, dv, slot, HEAD_MAX);
    if (T == 0) return 0;
    LC_CHECK(proj && q_out, "head_norm_write: null pointer");
    LC_CHECK(page_size > 0 || !slots, "head_norm_write: bad page size");
    const bool writes = nkv > 0 && slots && k_cache && v_cache;
    // without a cache to write, only the q heads are work
    const int per_token = nh + 2 * nkv;
    LC_CHECK((long long)T * per_token < (1ll << 31), "head_norm_write: too many heads");
    if (dt == DT_F32)
        head_norm_write_kernel<float><<<T * per_token, kWave, 0, stream>>>(
            (const float*)proj, nh, nkv, d, dv, slot, qw, kw, eps, head_scale, (float*)q_out,
            writes ? (float*)k_cache : nullptr, writes ? (float*)v_cache : nullptr, writes ? slots : nullptr,
            page_size > 0 ? page_size : 1, num_pages);
    else if (dt == DT_BF16)
        head_norm_write_kernel<bf16><<<T * per_token, kWave, 0, stream>>>(
            (const bf16*)proj, nh, nkv, d, dv, slot, qw, kw, eps, head_scale, (bf16*)q_out,
            writes ? (bf16*)k_cache : nullptr, writes ? (bf16*)v_cache : nullptr, writes ? slots : nullptr,
            page_size > 0 ? page_size : 1, num_pages);
    else
        LC_CHECK(false, "head_norm_write: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("head_norm_write");
    return 0;
}

// gate: 0 sigmoid, 1 silu
LC_API int lc_head_gate_norm(const float* o, const float* gates, int gate_cols, int gate_column, const float* weight,
                             int per_head, float eps, int gate, int T, int heads, int dim, void* out, int dt,
                             hipStream_t stream) {
    LC_CHECK(T >= 0 && heads > 0 && dim > 0 && gate_column >= 0 && gate_column + heads * dim <= gate_cols,
             "head_gate_norm: bad sizes");
    LC_CHECK(gate == 0 || gate == 1, "head_gate_norm: unknown gate %d", gate);
    if (T == 0) return 0;
    LC_CHECK(o && gates && weight && out, "head_gate_norm: null pointer");
    LC_CHECK((long long)T * heads < (1ll << 31), "head_gate_norm: too many heads");
    if (dt == DT_F32)
        head_gate_norm_kernel<float><<<T * heads, kWave, 0, stream>>>(o, gates, gate_cols, gate_column, weight, per_head,
                                                                      eps, gate, heads, dim, (float*)out);
    else if (dt == DT_BF16)
        head_gate_norm_kernel<bf16><<<T * heads, kWave, 0, stream>>>(o, gates, gate_cols, gate_column, weight, per_head,
                                                                     eps, gate, heads, dim, (bf16*)out);
    else
        LC_CHECK(false, "head_gate_norm: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("head_gate_norm");
    return 0;
}
