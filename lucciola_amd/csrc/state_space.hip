// The state-space mixer (Mamba-2's recurrence) around the framework's recurrence kernel.  Per head h of
// group g = h / (heads / groups), with the state S [N, dv] (float32, zeros at a sequence's start):
//   step = softplus(dt_h + dt_bias_h);   S <- exp(-exp(A_log_h) step) S + step B_g x_h^T;   y_h = S^T C_g + D_h x_h
// x, B and C pass a short causal convolution per channel (with a bias) and SiLU first.  That is the
// recurrence S <- diag(decay) S + write v^T, o = S^T read without a removal term, with decay = exp(-exp(A_log)
// step) in every key channel, write = step B, read = C, v = x: this file makes those three vectors a token
// from a step's float32 projections, and the read-out behind the scan:
//   y <- (o + D x) silu(z), divided by its root mean square in `parts` equal parts of the row, times a weight.
// Everything here is float32 arithmetic; only the read-out's result is rounded to the activation type.
#include "common.h"
#include "short_conv.h"

namespace lc {

__device__ __forceinline__ float ss_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float ss_softplus(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

// A thread per convolved entry.  proj [T, cols]: x (heads dv) | B (groups N) | C (groups N) | z (heads dv) | dt (heads);
// the first C = heads dv + 2 groups N columns pass the convolution.  Entry (t, i): i < heads dv is a channel of x;
// the others are (group, n) pairs, whose thread makes B and C at n and writes them for every head of the group with
// the head's own step and decay.  coef [3, T, heads N]; x_out [T, heads dv]
__global__ void state_space_prepare_kernel(const float* __restrict__ proj, int cols, int T, int heads, int groups,
                                           int N, int dv, const float* __restrict__ taps, const float* __restrict__ bias,
                                           int K, const float* __restrict__ tails, const float* __restrict__ dt_bias,
                                           const float* __restrict__ a_log, const int* __restrict__ tok_req,
                                           const int* __restrict__ q_offsets, const int* __restrict__ slot_ids,
                                           float* __restrict__ coef, float* __restrict__ x_out) {
    const int inner = heads * dv, C = inner + 2 * groups * N, per_token = inner + groups * N, per_group = heads / groups;
    const size_t total = (size_t)T * per_token, plane = (size_t)T * heads * N;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int t = (int)(idx / per_token), i = (int)(idx % per_token);
        const int r = tok_req[t];
        const int local = t - q_offsets[r];
        const float* tail = K > 1 ? tails + (size_t)slot_ids[r] * (K - 1) * C : nullptr;
        if (i < inner) {
            x_out[(size_t)t * inner + i] = ss_silu(short_conv(proj, cols, t, local, i, taps, K, tail, C) + bias[i]);
            continue;
        }
        const int g = (i - inner) / N, n = (i - inner) % N;
        const int cb = inner + g * N + n, cc = inner + groups * N + g * N + n;
        const float b = ss_silu(short_conv(proj, cols, t, local, cb, taps, K, tail, C) + bias[cb]);
        const float c = ss_silu(short_conv(proj, cols, t, local, cc, taps, K, tail, C) + bias[cc]);
        for (int k = 0; k < per_group; ++k) {
            const int head = g * per_group + k;
            const float step = ss_softplus(proj[(size_t)t * cols + C + inner + head] + dt_bias[head]);
            const size_t at = ((size_t)t * heads + head) * N + n;
            coef[at] = expf(-expf(a_log[head]) * step);
            coef[plane + at] = step * b;
            coef[2 * plane + at] = c;
        }
    }
}

// One workgroup per token and part of the row.  o, x float32 [T, n]; z float32: columns z_column .. + n of gates
// [T, gate_cols]; skip float32 [heads] (D); weight float32 [n]; the row is normed in `parts` equal parts.
template <typename T>
__global__ void state_space_readout_kernel(const float* __restrict__ o, const float* __restrict__ x,
                                           const float* __restrict__ gates, int gate_cols, int z_column,
                                           const float* __restrict__ skip, int dv, const float* __restrict__ weight,
                                           int parts, float eps, int n, T* __restrict__ out) {
    extern __shared__ float y[];
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    const int width = n / parts, first = blockIdx.y * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const int at = first + i;
        const float v = fmaf(skip[at / dv], x[t * n + at], o[t * n + at]) * ss_silu(gates[t * gate_cols + z_column + at]);
        y[i] = v;                       // a thread meets its own entries only
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[t * n + first + i] = from_f32<T>(y[i] * inv * weight[first + i]);
}

// out = a_scale a + b_scale b, float32 arithmetic
template <typename TA, typename TB>
__global__ void scaled_sum_kernel(const TA* __restrict__ a, float a_scale, const TB* __restrict__ b, float b_scale,
                                  float* __restrict__ out, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        out[i] = fmaf(b_scale, to_f32(b[i]), a_scale * to_f32(a[i]));
}

}  // namespace lc

using namespace lc;

LC_API int lc_state_space_prepare(const float* proj, int cols, int T, int heads, int groups, int N, int dv,
                                  const float* taps, const float* bias, int K, const float* tails, const float* dt_bias,
                                  const float* a_log, const int* tok_req, const int* q_offsets, const int* slot_ids,
                                  float* coef, float* x_out, hipStream_t stream) {
    LC_CHECK(T >= 0 && heads > 0 && groups > 0 && N > 0 && dv > 0 && heads % groups == 0, "state space prepare: bad sizes");
    LC_CHECK(cols == 2 * heads * dv + 2 * groups * N + heads, "state space prepare: %d columns do not fit the sizes", cols);
    LC_CHECK(K >= 1 && K <= SHORT_CONV_MAX_TAPS, "state space prepare: %d taps (1 to %d)", K, SHORT_CONV_MAX_TAPS);
    if (T == 0) return 0;
    LC_CHECK(proj && taps && bias && dt_bias && a_log && tok_req && q_offsets && slot_ids && coef && x_out && (K == 1 || tails),
             "state space prepare: null pointer");
    const size_t total = (size_t)T * (heads * dv + groups * N);
    const int blocks = (int)((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
    state_space_prepare_kernel<<<blocks, 256, 0, stream>>>(proj, cols, T, heads, groups, N, dv, taps, bias, K, tails, dt_bias,
                                                           a_log, tok_req, q_offsets, slot_ids, coef, x_out);
    LC_LAUNCH_CHECK("state_space_prepare");
    return 0;
}

LC_API int lc_state_space_readout(const float* o, const float* x, const float* gates, int gate_cols, int z_column,
                                  const float* skip, int heads, int dv, const float* weight, int parts, float eps, int T,
                                  void* out, int dt, hipStream_t stream) {
    const int n = heads * dv;
    LC_CHECK(T >= 0 && heads > 0 && dv > 0 && parts > 0 && n % parts == 0 && z_column >= 0 && z_column + n <= gate_cols,
             "state space readout: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(o && x && gates && skip && weight && out, "state space readout: null pointer");
    const int width = n / parts;
    const size_t lds = (size_t)width * sizeof(float);
    LC_CHECK(lds <= 48 * 1024, "state space readout: parts of %d entries are too long", width);
    LC_CHECK(parts <= 65535, "state space readout: too many parts (%d)", parts);
    const int threads = width >= 1024 ? 256 : (width >= 256 ? 128 : 64);
    const dim3 grid(T, parts);
    if (dt == DT_F32)
        state_space_readout_kernel<float><<<grid, threads, lds, stream>>>(o, x, gates, gate_cols, z_column, skip, dv, weight,
                                                                          parts, eps, n, (float*)out);
    else if (dt == DT_BF16)
        state_space_readout_kernel<bf16><<<grid, threads, lds, stream>>>(o, x, gates, gate_cols, z_column, skip, dv, weight,
                                                                         parts, eps, n, (bf16*)out);
    else
        LC_CHECK(false, "state space readout: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("state_space_readout");
    return 0;
}

// a [rows, n] of dtype dt_a, b likewise -> out float32
LC_API int lc_scaled_sum(const void* a, int dt_a, float a_scale, const void* b, int dt_b, float b_scale, float* out,
                         long long total, hipStream_t stream) {
    LC_CHECK(total >= 0, "scaled sum: bad size");
    if (total == 0) return 0;
    LC_CHECK(a && b && out, "scaled sum: null pointer");
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
#define LC_SS(TA, TB) scaled_sum_kernel<TA, TB><<<blocks, 256, 0, stream>>>((const TA*)a, a_scale, (const TB*)b, b_scale, out, (size_t)total)
    if (dt_a == DT_F32 && dt_b == DT_F32) LC_SS(float, float);
    else if (dt_a == DT_F32 && dt_b == DT_BF16) LC_SS(float, bf16);
    else if (dt_a == DT_BF16 && dt_b == DT_F32) LC_SS(bf16, float);
    else if (dt_a == DT_BF16 && dt_b == DT_BF16) LC_SS(bf16, bf16);
    else LC_CHECK(false, "scaled sum: unknown dtypes %d, %d", dt_a, dt_b);
#undef LC_SS
    LC_LAUNCH_CHECK("scaled_sum");
    return 0;
}
