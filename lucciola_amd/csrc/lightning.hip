// Lightning attention: linear attention with one decay per head.  Per head and request, with the state
// S [key, value] (float32, zeros at a sequence's start):
//   q = silu(W_q h), k = silu(W_k h), v = silu(W_v h);   S <- decay S + k v^T;   o = S^T q
// This file turns a step's float32 projections into the inputs of the framework's recurrence kernel
// (S <- diag(decay) S - removal (probe^T S) + write v^T, o = S^T read), of which lightning attention is
// the case decay = one number per head, probe = removal = 0, write = k, read = q.
#include "common.h"

namespace lc {

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }

// proj [T, cols]: q | k (heads x dk each) | v (heads x dv) | ...; coef [5, T, heads dk]; v_out [T, heads dv]
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
            coef[plane + at] = 0.f;
            coef[2 * plane + at] = 0.f;
            coef[3 * plane + at] = silu_f(row[nk + c]);
            coef[4 * plane + at] = silu_f(row[c]);
        } else {
            v_out[(size_t)t * nv + (c - nk)] = silu_f(row[2 * nk + (c - nk)]);
        }
    }
}

}  // namespace lc

using namespace lc;

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
