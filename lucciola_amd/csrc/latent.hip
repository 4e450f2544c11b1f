// Latent attention over a paged cache that keeps one row [c | k_r] per token: the latent c (R
// entries, RMS-normed) and a rotated key part k_r (rot entries) that all heads share.
//
// The query arrives in the latent's space, head by head [q_c | q_r] (q_c = W_uk^T q_plain, R
// entries; q_r the rotated part, rot entries), so that for every head
//   s_j = ([q_c | q_r] . [c_j | k_r,j]) * scale        over the keys j <= p, and j > p - window
//   P = softmax(s),   o = sum_j P_j c_j                (R entries; W_uv is applied afterwards)
// With a sink per head the softmax's denominator holds one more term, exp(sink): a key that has the
// score `sink` (not scaled) whatever the query, and no value.
// All heads of a token read the same rows.  Arithmetic is float32 throughout (scores, maximum,
// exponentials, sums, P.c); only loads and stores have the tensors' type.
//
// The order of the additions is a function of the query alone: its keys are taken in chunks of 64
// from its first visible key on, a key's score adds its entries in a fixed order, and a chunk's
// weighted rows are added key by key.  A token's result has the same bits in a prompt's portion
// and in a step of single tokens.
#include "common.h"

namespace lc {

constexpr int LA_THREADS = 256;
constexpr int LA_HEADS = 4;       // heads a workgroup serves together: one wave each for the softmax
constexpr int LA_KEYS = 64;       // keys of a chunk
constexpr int LA_DIMS = 8;        // output entries a thread sums: R <= LA_THREADS * LA_DIMS

// ------------------------------------------------------------------------------ prologue
// One workgroup per token.  From the token's rows of two tensors, [q heads ...] and [c' | k_r | ...] (the
// same fused projection at two columns, or the queries from a product of their own):
//   c = c' / sqrt(mean(c'^2) + eps) * w  and  rot(k_r) go to the token's cache row (slot >= 0);
//   rot(q_r) of every head goes to qa[t][h][R ...].
// Rotation of the first `rd` entries of a part: interleaved pairs (2i, 2i + 1) or halves
// (i, i + rd/2), by the angle whose cosine and sine are table[p][i] and table[p][rd/2 + i].
template <typename T>
__global__ __launch_bounds__(LA_THREADS) void latent_prepare_kernel(
    const T* __restrict__ q, long long ldq, const T* __restrict__ kv, long long ld, int H, int dim, int rot, int R,
    const float* __restrict__ w,
    float eps, const int* __restrict__ positions, const float* __restrict__ table, int rd, int interleaved,
    T* __restrict__ cache, const int* __restrict__ slots, T* __restrict__ qa) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const T* row = q + (size_t)t * ldq;
    const T* down = kv + (size_t)t * ld;
    const int Dk = R + rot;
    const long long slot = slots ? slots[t] : -1;
    T* mine = slot >= 0 ? cache + slot * Dk : nullptr;
    float ss = 0.f;
    for (int i = tid; i < R; i += LA_THREADS) {
        const float v = to_f32(down[i]);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)R + eps);
    if (mine)
        for (int i = tid; i < R; i += LA_THREADS) mine[i] = from_f32<T>(to_f32(down[i]) * inv * w[i]);
    const float* cs = table ? table + (size_t)positions[t] * rd : nullptr;
    const int half = rd / 2;
    // entry e of a rotated part, from the part's raw entries
    auto turned = [&](const T* part, int e) -> float {
        const float own = to_f32(part[e]);
        if (!cs || e >= rd) return own;
        int pair, other;
        bool first;
        if (interleaved) { pair = e >> 1; first = (e & 1) == 0; other = e ^ 1; }
        else { pair = e < half ? e : e - half; first = e < half; other = first ? e + half : e - half; }
        const float c = cs[pair], s = cs[half + pair], o = to_f32(part[other]);
        // (u, v) -> (u c - v s, v c + u s)
        return first ? __fsub_rn(__fmul_rn(own, c), __fmul_rn(o, s)) : __fadd_rn(__fmul_rn(own, c), __fmul_rn(o, s));
    };
    if (mine)
        for (int e = tid; e < rot; e += LA_THREADS) mine[R + e] = from_f32<T>(turned(down + R, e));
    for (int i = tid; i < H * rot; i += LA_THREADS) {
        const int h = i / rot, e = i - h * rot;
        qa[((size_t)t * H + h) * Dk + R + e] = from_f32<T>(turned(row + (size_t)h * (dim + rot) + dim, e));
    }
}

// ------------------------------------------------------------------------------ attention
// One workgroup per token and LA_HEADS heads.  LDS: the heads' queries (scaled), a chunk's
// scores and weights, the chunk's cache rows.
template <typename T, bool VEC>
__global__ __launch_bounds__(LA_THREADS) void latent_attention_kernel(
    const T* __restrict__ qa, int H, int R, int rot, const T* __restrict__ cache,
    const int* __restrict__ tok_req, const int* __restrict__ positions, const int* __restrict__ block_table,
    int max_blocks, int page_size, float scale, int window, const float* __restrict__ sink, T* __restrict__ out) {
    extern __shared__ float smem[];
    const int Dk = R + rot, Dp = (Dk + 3) & ~3;
    float* qs = smem;                                   // [LA_HEADS][Dp]
    float* ps = qs + LA_HEADS * Dp;                     // [LA_HEADS][LA_KEYS]
    float* alpha_s = ps + LA_HEADS * LA_KEYS;           // [LA_HEADS]
    float* l_s = alpha_s + LA_HEADS;                    // [LA_HEADS]
    int* rows = reinterpret_cast<int*>(l_s + LA_HEADS); // [LA_KEYS]: page * page_size + offset of the chunk's keys
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int t = blockIdx.x, h0 = blockIdx.y * LA_HEADS, heads = min(LA_HEADS, H - h0);
    const int p = positions[t];
    const int* table = block_table + (size_t)tok_req[t] * max_blocks;
    const int j_lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;

    for (int i = tid; i < LA_HEADS * Dp; i += LA_THREADS) {
        const int hh = i / Dp, e = i - hh * Dp;
        qs[i] = (hh < heads && e < Dk) ? to_f32(qa[((size_t)t * H + h0 + hh) * Dk + e]) * scale : 0.f;
    }
    float m_run = -INFINITY, l_run = 0.f;               // of head `wave`, the same in all its lanes
    if (sink && wave < heads) {                         // the sink: seen before the first key, weight exp(0)
        m_run = sink[h0 + wave];
        l_run = 1.f;
    }
    float acc[LA_HEADS][LA_DIMS];
#pragma unroll
    for (int hh = 0; hh < LA_HEADS; ++hh)
#pragma unroll
        for (int x = 0; x < LA_DIMS; ++x) acc[hh][x] = 0.f;

    const int kk = tid >> 2, piece = tid & 3;           // scores: four lanes a key
    for (int c0 = j_lo; c0 <= p; c0 += LA_KEYS) {
        const int count = min(LA_KEYS, p - c0 + 1);
        __syncthreads();                                // the chunk before has been read; qs is written
        if (tid < LA_KEYS) {
            const int j = c0 + min(tid, count - 1);
            rows[tid] = table[j / page_size] * page_size + j % page_size;
        }
        __syncthreads();
        {
            const T* krow = cache + (size_t)rows[kk] * Dk;
            float dot[LA_HEADS];
#pragma unroll
            for (int hh = 0; hh < LA_HEADS; ++hh) dot[hh] = 0.f;
            if constexpr (VEC) {
                for (int e = piece * 4; e < Dk; e += 16) {
                    float k4[4];
                    load4(k4, krow + e);
#pragma unroll
                    for (int hh = 0; hh < LA_HEADS; ++hh) {
                        const float4 q4 = *reinterpret_cast<const float4*>(qs + hh * Dp + e);
                        float s = dot[hh];
                        s = fmaf(q4.x, k4[0], s);
                        s = fmaf(q4.y, k4[1], s);
                        s = fmaf(q4.z, k4[2], s);
                        s = fmaf(q4.w, k4[3], s);
                        dot[hh] = s;
                    }
                }
            } else {
                for (int e = piece; e < Dk; e += 4) {
                    const float kv = to_f32(krow[e]);
#pragma unroll
                    for (int hh = 0; hh < LA_HEADS; ++hh) dot[hh] = fmaf(qs[hh * Dp + e], kv, dot[hh]);
                }
            }
#pragma unroll
            for (int hh = 0; hh < LA_HEADS; ++hh) {
                float s = dot[hh];
                s = __fadd_rn(s, __shfl_xor(s, 1, kWave));
                s = __fadd_rn(s, __shfl_xor(s, 2, kWave));
                if (piece == 0) ps[hh * LA_KEYS + kk] = kk < count ? s : -INFINITY;
            }
        }
        __syncthreads();
        {   // wave w: the softmax step of head w over the chunk's 64 scores
            const float s = ps[wave * LA_KEYS + lane];
            const float m_new = fmaxf(m_run, wave_max(s));
            const float pj = lane < count ? expf(s - m_new) : 0.f;
            const float alpha = expf(m_run - m_new);    // 0 for the first chunk (m_run = -inf)
            l_run = fmaf(l_run, alpha, wave_sum(pj));
            m_run = m_new;
            ps[wave * LA_KEYS + lane] = pj;
            if (lane == 0) alpha_s[wave] = alpha;
        }
        __syncthreads();
#pragma unroll
        for (int hh = 0; hh < LA_HEADS; ++hh) {
            const float alpha = alpha_s[hh];
#pragma unroll
            for (int x = 0; x < LA_DIMS; ++x) acc[hh][x] = __fmul_rn(acc[hh][x], alpha);
        }
#pragma unroll
        for (int x = 0; x < LA_DIMS; ++x) {
            const int d = tid + LA_THREADS * x;
            if (d < R) {
#pragma unroll 4
                for (int j = 0; j < count; ++j) {
                    const float v = to_f32(cache[(size_t)rows[j] * Dk + d]);
#pragma unroll
                    for (int hh = 0; hh < LA_HEADS; ++hh) acc[hh][x] = fmaf(ps[hh * LA_KEYS + j], v, acc[hh][x]);
                }
            }
        }
    }
    if (lane == 0) l_s[wave] = l_run;
    __syncthreads();
#pragma unroll
    for (int hh = 0; hh < LA_HEADS; ++hh)
        if (hh < heads) {
            const float l = l_s[hh];
#pragma unroll
            for (int x = 0; x < LA_DIMS; ++x) {
                const int d = tid + LA_THREADS * x;
                if (d < R) out[((size_t)t * H + h0 + hh) * R + d] = from_f32<T>(acc[hh][x] / l);
            }
        }
}

static size_t latent_attention_lds(int R, int rot) {
    const int Dp = (R + rot + 3) & ~3;
    return sizeof(float) * (LA_HEADS * Dp + LA_HEADS * LA_KEYS + 2 * LA_HEADS) + sizeof(int) * LA_KEYS;
}

}  // namespace lc

using namespace lc;

// q [T, ldq]: [H x (dim | rot) | ...]; kv [T, ld]: [R | rot | ...]; cache [slots, R + rot]; qa [T, H, R + rot].
// table: float32 [positions, rd] (cosines, then sines) or null; rd <= rot.
LC_API int lc_latent_prepare(const void* q, long long ldq, const void* proj, int dt, long long ld, int T, int H,
                             int dim, int rot, int R,
                             const float* w, float eps, const int* positions, const float* table, int rd,
                             int interleaved, void* cache, const int* slots, void* qa, hipStream_t stream) {
    LC_CHECK(T >= 0 && H > 0 && dim >= 0 && rot >= 0 && R > 0, "latent prepare: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(q && proj && w && qa, "latent prepare: null pointer");
    LC_CHECK(ld >= (long long)R + rot && ldq >= (long long)H * (dim + rot),
             "latent prepare: rows of %lld and %lld entries are too short", ldq, ld);
    LC_CHECK(!table || (positions && rd > 0 && rd % 2 == 0 && rd <= rot), "latent prepare: %d rotated entries in a part of %d", rd, rot);
    LC_CHECK((cache == nullptr) == (slots == nullptr), "latent prepare: cache and slots come together");
    if (dt == DT_F32)
        latent_prepare_kernel<float><<<T, LA_THREADS, 0, stream>>>((const float*)q, ldq, (const float*)proj, ld, H, dim, rot, R, w, eps, positions,
                                                                  table, rd, interleaved, (float*)cache, slots, (float*)qa);
    else if (dt == DT_BF16)
        latent_prepare_kernel<bf16><<<T, LA_THREADS, 0, stream>>>((const bf16*)q, ldq, (const bf16*)proj, ld, H, dim, rot, R, w, eps, positions,
                                                                 table, rd, interleaved, (bf16*)cache, slots, (bf16*)qa);
    else
        LC_CHECK(false, "latent prepare: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("latent_prepare");
    return 0;
}

// qa [T, H, R + rot], cache [slots, R + rot] -> out [T, H, R]
LC_API int lc_latent_attention(const void* qa, int dt, int T, int H, int R, int rot, const void* cache,
                               const int* tok_req, const int* positions, const int* block_table, int max_blocks,
                               int page_size, float scale, int window, const float* sink, void* out,
                               hipStream_t stream) {
    LC_CHECK(T >= 0 && H > 0 && R > 0 && rot >= 0 && page_size > 0 && max_blocks > 0, "latent attention: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(qa && cache && tok_req && positions && block_table && out, "latent attention: null pointer");
    LC_CHECK(R <= LA_THREADS * LA_DIMS, "latent attention: a latent of %d entries is above the supported %d", R,
             LA_THREADS * LA_DIMS);
    LC_CHECK((H + LA_HEADS - 1) / LA_HEADS <= 65535, "latent attention: too many heads (%d)", H);
    const size_t lds = latent_attention_lds(R, rot);
    LC_CHECK(lds <= 64 * 1024, "latent attention: rows of %d entries do not fit the workgroup's memory", R + rot);
    const dim3 grid(T, (H + LA_HEADS - 1) / LA_HEADS);
    const bool vec = (R + rot) % 4 == 0 && (uintptr_t)cache % 16 == 0;
#define LC_LA_LAUNCH(TYPE, VEC)                                                                                   \
    latent_attention_kernel<TYPE, VEC><<<grid, LA_THREADS, lds, stream>>>((const TYPE*)qa, H, R, rot, (const TYPE*)cache, \
        tok_req, positions, block_table, max_blocks, page_size, scale, window, sink, (TYPE*)out)
    if (dt == DT_F32) {
        if (vec) LC_LA_LAUNCH(float, true); else LC_LA_LAUNCH(float, false);
    } else if (dt == DT_BF16) {
        if (vec) LC_LA_LAUNCH(bf16, true); else LC_LA_LAUNCH(bf16, false);
    } else {
        LC_CHECK(false, "latent attention: unknown dtype %d", dt);
    }
#undef LC_LA_LAUNCH
    LC_LAUNCH_CHECK("latent_attention");
    return 0;
}
