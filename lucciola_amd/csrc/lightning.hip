// Lightning attention: linear attention with one decay per head.  Per head and request, with the state
// S [key, value] (float32, zeros at a sequence's start):
//   q = silu(W_q h), k = silu(W_k h), v = silu(W_v h);   S <- decay S + k v^T;   o = S^T q
// This file turns a step's float32 projections into the inputs of the framework's recurrence kernel
// without its removal term (S <- diag(decay) S + write v^T, o = S^T read: three vectors a token), of
// which lightning attention is the case decay = one number per head, write = k, read = q.
#include "common.h"

namespace lc {

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

// proj [T, cols]: q | k (heads x dk each) | v (heads x dv) | ...; coef [3, T, heads dk]; v_out [T, heads dv]
__global__ void lightning_prepare_kernel(const float* __restrict__ proj, int cols, int T, int heads, int dk, int dv,
                                         const float* __restrict__ decay, float* __restrict__ coef,
                                         float* __restrict__ v_out) {
    const int nk = heads * dk, nv = heads * dv;
    const size_t plane = (size_t)T * nk;
    const size_t total = (size_t)T * (nk + nv);
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const int t = (int)(idx / (nk + nv)), c = (int)(idx % (nk + nv));
        const float* row = proj + (size_t)t * cols;
        if (c < nk) {
            const size_t at = (size_t)t * nk + c;
            coef[at] = decay[c / dk];
            coef[plane + at] = silu_f(row[nk + c]);
            coef[2 * plane + at] = silu_f(row[c]);
        } else {
            v_out[(size_t)t * nv + (c - nk)] = silu_f(row[2 * nk + (c - nk)]);
        }
    }
}

// One workgroup per token: all heads' read-outs together divided by their common root mean square, times
// a weight, times sigmoid(gate); o, gates and the weight float32, the result in the activation type.
template <typename T>
__global__ void lightning_readout_kernel(const float* __restrict__ o, const float* __restrict__ gates, int gate_cols,
                                         int gate_column, const float* __restrict__ weight, float eps, int n,
                                         T* __restrict__ out) {
    __shared__ float scratch[16];
    const float* x = o + (size_t)blockIdx.x * n;
    const float* g = gates + (size_t)blockIdx.x * gate_cols + gate_column;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(x[i], x[i], ss);
    const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
    T* dst = out + (size_t)blockIdx.x * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        dst[i] = from_f32<T>(x[i] * inv * weight[i] / (1.f + expf(-g[i])));
}

}  // namespace lc

using namespace lc;

// o float32 [T, n]; gates float32 [T, gate_cols], the row's n gates from gate_column on; weight float32 [n]
LC_API int lc_lightning_readout(const float* o, const float* gates, int gate_cols, int gate_column, const float* weight,
                                float eps, int T, int n, void* out, int dt, hipStream_t stream) {
    LC_CHECK(T >= 0 && n > 0 && gate_column >= 0 && gate_column + n <= gate_cols, "lightning readout: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(o && gates && weight && out, "lightning readout: null pointer");
    const int threads = n >= 2048 ? 512 : (n >= 512 ? 256 : (n >= 128 ? 128 : 64));
    if (dt == DT_F32)
        lightning_readout_kernel<float><<<T, threads, 0, stream>>>(o, gates, gate_cols, gate_column, weight, eps, n, (float*)out);
    else if (dt == DT_BF16)
        lightning_readout_kernel<bf16><<<T, threads, 0, stream>>>(o, gates, gate_cols, gate_column, weight, eps, n, (bf16*)out);
    else
        LC_CHECK(false, "lightning readout: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("lightning_readout");
    return 0;
}

LC_API int lc_lightning_prepare(const float* proj, int cols, int T, int heads, int dk, int dv, const float* decay,
                                float* coef, float* v_out, hipStream_t stream) {
    LC_CHECK(T >= 0 && heads > 0 && dk > 0 && dv > 0 && cols >= heads * (2 * dk + dv), "lightning prepare: bad sizes");
    if (T == 0) return 0;
    LC_CHECK(proj && decay && coef && v_out, "lightning prepare: null pointer");
    const size_t total = (size_t)T * heads * (dk + dv);
    const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
    lightning_prepare_kernel<<<blocks, 256, 0, stream>>>(proj, cols, T, heads, dk, dv, decay, coef, v_out);
    LC_LAUNCH_CHECK("lightning_prepare");
    return 0;
}
