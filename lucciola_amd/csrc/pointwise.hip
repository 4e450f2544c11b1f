// Element-wise kernels of the parts that came after the first architecture: the Dynamic Tanh
// norm (with the residual addition folded in, as the RMSNorm kernel has it), a vector added to
// every row of the residual stream, and the activations of the two-matrix feed-forwards.
// All arithmetic is float32; only loads and stores have the tensors' types.
//   dynamic tanh   y = tanh(alpha v) w + b,  v = h (+ delta)
//   gelu (tanh)    0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
//   relu squared   max(z, 0)^2
//   xIELU          z > 0: a z^2 + z/2;  z <= 0: b (e^z - 1 - z) + z/2
// and the token shift: what a mixer reads of token t becomes x_t + (x_(t-1) - x_t) mix, the row before
// a step's first token coming from the request's state.
#include "common.h"

#include "activations.h"

namespace lc {

// One workgroup per output row r; src row = rows ? rows[r] : r.
//   v = h[src] (+ delta[src]);  if (write_h) h[src] = v;  out[r] = tanh(alpha v) w + b
template <typename T>
__global__ void dynamic_tanh_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                    const int* __restrict__ rows, const float* __restrict__ w,
                                    const float* __restrict__ b, float alpha, T* __restrict__ out, int n,
                                    int write_h) {
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    float* hr = h + (size_t)src * n;
    const T* dr = delta ? delta + (size_t)src * n : nullptr;
    T* o = out + (size_t)r * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = hr[i];
        if (dr) {
            v += to_f32(dr[i]);
            if (write_h) hr[i] = v;
        }
        o[i] = from_f32<T>(fmaf(tanhf(alpha * v), w[i], b[i]));
    }
}

// h[t] += delta[t] (+ more[t]) + vec, for every row t
template <typename T>
__global__ void stream_add_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                  const float* __restrict__ more, const float* __restrict__ vec, int n,
                                  size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        float v = h[idx];
        if (delta) v += to_f32(delta[idx]);
        if (more) v += more[idx];
        h[idx] = v + vec[idx % n];
    }
}

template <typename T>
__global__ void activation_kernel(T* __restrict__ x, int kind, float a, float b, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x) {
        const float z = to_f32(x[idx]);
        x[idx] = from_f32<T>(kind == ACT_XIELU ? xielu(z, a, b) : activate(z, kind));
    }
}

__global__ void scale_kernel(float* __restrict__ x, float factor, size_t total) {
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (size_t)gridDim.x * blockDim.x)
        x[idx] *= factor;
}

// One workgroup per token t of request r = tok_req[t]:  y[t] = x[t] + (before - x[t]) mix, with before =
// x[t - 1], or, for the request's first token of the step, the row that state[slot] holds (what the
// request's last token left there; zeros at a sequence's start).  The first token's workgroup, the only
// one that reads the state, also writes the request's last row of this step into it: each thread the
// entries it has read itself.
template <typename T>
__global__ void token_shift_kernel(const T* __restrict__ x, const float* __restrict__ mix, float* __restrict__ state,
                                   const int* __restrict__ tok_req, const int* __restrict__ q_offsets,
                                   const int* __restrict__ slot_ids, T* __restrict__ y, int n) {
    const int t = blockIdx.x, r = tok_req[t];
    const int first = q_offsets[r], last = q_offsets[r + 1] - 1;
    const T* xr = x + (size_t)t * n;
    T* yr = y + (size_t)t * n;
    if (t == first) {
        float* st = state + (size_t)slot_ids[r] * n;
        const T* xl = x + (size_t)last * n;
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const float own = to_f32(xr[i]), before = st[i];
            yr[i] = from_f32<T>(fmaf(before - own, mix[i], own));
            st[i] = to_f32(xl[i]);
        }
    } else {
        const T* xb = xr - n;
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const float own = to_f32(xr[i]), before = to_f32(xb[i]);
            yr[i] = from_f32<T>(fmaf(before - own, mix[i], own));
        }
    }
}

// The same with the norm in front, one kernel: v = h (+ delta) goes to h_out; u_t = v_t / sqrt(mean(v_t^2) +
// eps) * g (one number g for all entries);  y[t] = u_t + (u_(t-1) - u_t) mix.  The state keeps u of a
// request's last token in float32.  A workgroup norms its own row and the row before it (the first
// token's workgroup: its own and the request's last of this step, for the state), so no workgroup waits
// for another.
template <typename T, typename TD>
__global__ void rms_shift_kernel(const float* __restrict__ h, const TD* __restrict__ delta, float* __restrict__ h_out,
                                 float g, float eps, const float* __restrict__ mix, float* __restrict__ state,
                                 const int* __restrict__ tok_req, const int* __restrict__ q_offsets,
                                 const int* __restrict__ slot_ids, T* __restrict__ y, int n) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, r = tok_req[t];
    const int first = q_offsets[r], last = q_offsets[r + 1] - 1;
    const bool head = t == first;
    const int other = head ? last : t - 1;          // the second row this workgroup norms
    const float* hr = h + (size_t)t * n;
    const float* ho = h + (size_t)other * n;
    const TD* dr = delta ? delta + (size_t)t * n : nullptr;
    const TD* dn = delta ? delta + (size_t)other * n : nullptr;
    float ss_own = 0.f, ss_other = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = hr[i], u = ho[i];
        if (delta) { v += to_f32(dr[i]); u += to_f32(dn[i]); }
        ss_own = fmaf(v, v, ss_own);
        ss_other = fmaf(u, u, ss_other);
    }
    ss_own = block_sum(ss_own, scratch);
    ss_other = other == t ? ss_own : block_sum(ss_other, scratch);      // a lone token: one row, one sum
    const float inv_own = g / sqrtf(ss_own / (float)n + eps), inv_other = g / sqrtf(ss_other / (float)n + eps);
    float* st = head ? state + (size_t)slot_ids[r] * n : nullptr;
    float* out_h = h_out + (size_t)t * n;
    T* yr = y + (size_t)t * n;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = hr[i], u = ho[i];
        if (delta) { v += to_f32(dr[i]); u += to_f32(dn[i]); }
        out_h[i] = v;
        const float own = v * inv_own, second = u * inv_other;
        const float before = head ? st[i] : second;
        yr[i] = from_f32<T>(fmaf(before - own, mix[i], own));
        if (head) st[i] = second;
    }
}

static int blocks_for(size_t total) { return (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192); }

}  // namespace lc

using namespace lc;

LC_API int lc_dynamic_tanh(float* h, const void* delta, const int* rows, const float* w, const float* b,
                           float alpha, void* out, int dt, int R, int n, int write_h, hipStream_t stream) {
    LC_CHECK(R >= 0 && n > 0, "dynamic_tanh: bad sizes R=%d n=%d", R, n);
    if (R == 0) return 0;
    LC_CHECK(h && w && b && out, "dynamic_tanh: null pointer");
    LC_CHECK(!(rows && write_h), "dynamic_tanh: gathered rows cannot be written back");
    // a row's entries are independent: with few rows, as many threads a row as it has pairs of
    // entries, so that no thread walks the row load after load
    const int threads = (R <= 256 && n >= 2048) ? 1024 : (n >= 512 ? 256 : (n >= 128 ? 128 : 64));
    if (dt == DT_F32)
        dynamic_tanh_kernel<float><<<R, threads, 0, stream>>>(h, (const float*)delta, rows, w, b, alpha, (float*)out, n, write_h);
    else if (dt == DT_BF16)
        dynamic_tanh_kernel<bf16><<<R, threads, 0, stream>>>(h, (const bf16*)delta, rows, w, b, alpha, (bf16*)out, n, write_h);
    else
        LC_CHECK(false, "dynamic_tanh: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("dynamic_tanh");
    return 0;
}

LC_API int lc_stream_add(float* h, const void* delta, int dt, const float* more, const float* vec, int T, int n,
                         hipStream_t stream) {
    LC_CHECK(T >= 0 && n > 0, "stream_add: bad sizes T=%d n=%d", T, n);
    if (T == 0) return 0;
    LC_CHECK(h && vec, "stream_add: null pointer");
    const size_t total = (size_t)T * n;
    if (dt == DT_F32)
        stream_add_kernel<float><<<blocks_for(total), 256, 0, stream>>>(h, (const float*)delta, more, vec, n, total);
    else if (dt == DT_BF16)
        stream_add_kernel<bf16><<<blocks_for(total), 256, 0, stream>>>(h, (const bf16*)delta, more, vec, n, total);
    else
        LC_CHECK(false, "stream_add: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("stream_add");
    return 0;
}

// kind: 1 gelu (tanh form), 2 relu squared, 5 xIELU with its two numbers (a, b); in place
LC_API int lc_activation(void* x, int dt, int kind, float a, float b, long long total, hipStream_t stream) {
    LC_CHECK(total >= 0 && (kind == ACT_GELU_TANH || kind == ACT_RELU_SQUARED || kind == ACT_XIELU),
             "activation: bad arguments");
    if (total == 0) return 0;
    LC_CHECK(x, "activation: null pointer");
    if (dt == DT_F32)
        activation_kernel<float><<<blocks_for((size_t)total), 256, 0, stream>>>((float*)x, kind, a, b, (size_t)total);
    else if (dt == DT_BF16)
        activation_kernel<bf16><<<blocks_for((size_t)total), 256, 0, stream>>>((bf16*)x, kind, a, b, (size_t)total);
    else
        LC_CHECK(false, "activation: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("activation");
    return 0;
}

// x float32, in place: x *= factor
LC_API int lc_scale(float* x, float factor, long long total, hipStream_t stream) {
    LC_CHECK(total >= 0, "scale: bad size");
    if (total == 0) return 0;
    LC_CHECK(x, "scale: null pointer");
    scale_kernel<<<blocks_for((size_t)total), 256, 0, stream>>>(x, factor, (size_t)total);
    LC_LAUNCH_CHECK("scale");
    return 0;
}

static int shift_threads(int n) { return n >= 2048 ? 512 : (n >= 512 ? 256 : (n >= 128 ? 128 : 64)); }

// x, y [T, n] of dtype dt; mix float32 [n]; state float32 [slots, n]; tok_req [T], q_offsets [R + 1],
// slot_ids [R].  Every request of the batch must have a token in it (q_offsets strictly rising).
LC_API int lc_token_shift(const void* x, int dt, const float* mix, float* state, const int* tok_req,
                          const int* q_offsets, const int* slot_ids, void* y, int T, int n, hipStream_t stream) {
    LC_CHECK(T >= 0 && n > 0, "token_shift: bad sizes T=%d n=%d", T, n);
    if (T == 0) return 0;
    LC_CHECK(x && mix && state && tok_req && q_offsets && slot_ids && y && x != y, "token_shift: null or aliased pointer");
    if (dt == DT_F32)
        token_shift_kernel<float><<<T, shift_threads(n), 0, stream>>>((const float*)x, mix, state, tok_req, q_offsets,
                                                                     slot_ids, (float*)y, n);
    else if (dt == DT_BF16)
        token_shift_kernel<bf16><<<T, shift_threads(n), 0, stream>>>((const bf16*)x, mix, state, tok_req, q_offsets,
                                                                    slot_ids, (bf16*)y, n);
    else
        LC_CHECK(false, "token_shift: unknown dtype %d", dt);
    LC_LAUNCH_CHECK("token_shift");
    return 0;
}

// h, h_out float32 [T, n] (different tensors); delta [T, n] of dtype dt_delta or null; y [T, n] of dtype dt
LC_API int lc_rms_shift(const float* h, const void* delta, int dt_delta, float* h_out, float g, float eps,
                        const float* mix, float* state, const int* tok_req, const int* q_offsets,
                        const int* slot_ids, void* y, int dt, int T, int n, hipStream_t stream) {
    LC_CHECK(T >= 0 && n > 0, "rms_shift: bad sizes T=%d n=%d", T, n);
    if (T == 0) return 0;
    LC_CHECK(h && h_out && h != h_out && mix && state && tok_req && q_offsets && slot_ids && y,
             "rms_shift: null or aliased pointer");
    const int threads = shift_threads(n);
#define LC_RS(TO, TD)                                                                                          \
    rms_shift_kernel<TO, TD><<<T, threads, 0, stream>>>(h, (const TD*)delta, h_out, g, eps, mix, state, tok_req, \
                                                        q_offsets, slot_ids, (TO*)y, n)
    if (dt == DT_F32 && (dt_delta == DT_F32 || !delta)) LC_RS(float, float);
    else if (dt == DT_F32 && dt_delta == DT_BF16) LC_RS(float, bf16);
    else if (dt == DT_BF16 && (dt_delta == DT_BF16 || !delta)) LC_RS(bf16, bf16);
    else if (dt == DT_BF16 && dt_delta == DT_F32) LC_RS(bf16, float);
    else LC_CHECK(false, "rms_shift: unknown dtypes %d, %d", dt, dt_delta);
#undef LC_RS
    LC_LAUNCH_CHECK("rms_shift");
    return 0;
}
