// Mixers that keep a matrix of state per head and request: the delta-rule recurrence and what
// turns a layer's projections into its inputs.  Everything here is float32.
//
// The recurrence, per head, with the state S [key, value] and per token the vectors decay,
// probe, removal, write, read over the key channels and the value v:
//     S <- diag(decay) S - removal (probe^T S) + write v^T        (probe^T S: of S as the last token left it)
//     o  = S^T read
// A column of S (one value channel) never meets another, so the work is shared out by columns:
// a workgroup owns 16 columns of one head of one request and walks the request's tokens in
// order; a column belongs to 16 neighbouring lanes (a DPP row, so the two sums over the key rows
// that a token needs never leave the registers), each holding a run of the key rows.  The tokens'
// vectors come through LDS a stage of tokens at a time, the next stage loading meanwhile.
//
// The two delta rules differ in how the five vectors are made:
//   generalized   decay = exp(-c sigmoid(W2 tanh(x1) + w0)), a = sigmoid(xa + ba), u = k / sqrt(|k|^2 + e):
//                 probe = u, removal = a u, write = k, read = r
//   gated         q, k, v through a short causal convolution per channel and silu; q, k unit vectors,
//                 q times key_dim^-1/2; g = exp(-exp(A) softplus(xg + bg)), beta = sigmoid(xb):
//                 decay = g, probe = g k, removal = beta k, write = beta k, read = q
#include "common.h"

#include "activations.h"

namespace lc {

constexpr int DELTA_MAX_KEY = 256;
constexpr int DELTA_PER_LANE = DELTA_MAX_KEY / kWave;
constexpr int DELTA_MAX_INNER = 1024;
constexpr int CONV_MAX_TAPS = 16;

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// One wave per (token, head).  proj [T, 5 n + inner]: r | k | v | gate | removal | decay_in.
__global__ __launch_bounds__(kWave) void general_delta_prepare_kernel(
    const float* __restrict__ proj, int T, int heads, int dim, int inner, const float* __restrict__ decay_out,
    const float* __restrict__ decay_bias, const float* __restrict__ removal_bias, float unit_eps, float decay_scale,
    float* __restrict__ coef, float* __restrict__ v_out) {
    __shared__ float hidden[DELTA_MAX_INNER];
    const int t = blockIdx.x / heads, head = blockIdx.x % heads, lane = threadIdx.x;
    const int n = heads * dim;
    const size_t cols = (size_t)5 * n + inner;
    const float* row = proj + (size_t)t * cols;
    for (int j = lane; j < inner; j += kWave) hidden[j] = tanhf(row[(size_t)5 * n + j]);
    __syncthreads();
    float k[DELTA_PER_LANE], ss = 0.f;
#pragma unroll
    for (int e = 0; e < DELTA_PER_LANE; ++e) {
        const int i = lane + kWave * e;
        k[e] = i < dim ? row[n + head * dim + i] : 0.f;
        ss = fmaf(k[e], k[e], ss);
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) + unit_eps);
    const size_t plane = (size_t)T * n;
#pragma unroll
    for (int e = 0; e < DELTA_PER_LANE; ++e) {
        const int i = lane + kWave * e;
        if (i >= dim) continue;
        const int c = head * dim + i;
        float z = decay_bias[c];
        const float* w2 = decay_out + (size_t)c * inner;
        for (int j = 0; j < inner; ++j) z = fmaf(hidden[j], w2[j], z);
        const float decay = expf(-decay_scale * sigmoid(z));
        const float a = sigmoid(row[(size_t)4 * n + c] + removal_bias[c]);
        const float u = k[e] * inv;
        const size_t at = (size_t)t * n + c;
        coef[at] = decay;
        coef[plane + at] = u;
        coef[2 * plane + at] = a * u;
        coef[3 * plane + at] = k[e];
        coef[4 * plane + at] = row[c];
        v_out[at] = row[(size_t)2 * n + c];
    }
}

// Channel c of token t through the convolution: sum_j taps[c, K - 1 - j] x[t - j, c], where an input
// from before the step comes from the request's tail (its last K - 1 inputs, oldest first).
// KT: the number of taps where it is known when the kernel is built (all of a channel's loads are
// then asked for together), 0: whatever K says.
template <int KT>
__device__ __forceinline__ float conv_at(const float* __restrict__ proj, size_t cols, int t, int local, int c,
                                         const float* __restrict__ taps, int K, const float* __restrict__ tail, int C) {
    float y = 0.f;
    if constexpr (KT > 0) {
        float x[KT], w[KT];
#pragma unroll
        for (int j = 0; j < KT; ++j) {
            x[j] = j <= local ? proj[(size_t)(t - j) * cols + c] : tail[(size_t)((KT - 1) - (j - local)) * C + c];
            w[j] = taps[(size_t)c * KT + (KT - 1 - j)];
        }
#pragma unroll
        for (int j = 0; j < KT; ++j) y = fmaf(w[j], x[j], y);
    } else {
        for (int j = 0; j < K; ++j) {
            const float x = j <= local ? proj[(size_t)(t - j) * cols + c]
                                       : tail[(size_t)((K - 1) - (j - local)) * C + c];
            y = fmaf(taps[(size_t)c * K + (K - 1 - j)], x, y);
        }
    }
    return y;
}

// One wave per (token, head).  proj [T, C + nv + 2 heads]: q | k | v | gate | beta | rate.
template <int KT>
__global__ __launch_bounds__(kWave) void gated_delta_prepare_kernel(
    const float* __restrict__ proj, int T, int heads, int kv_heads, int dk, int dv, int K,
    const float* __restrict__ taps, const float* __restrict__ tails, const float* __restrict__ rate_log,
    const float* __restrict__ rate_bias, float unit_eps, const int* __restrict__ tok_req,
    const int* __restrict__ q_offsets, const int* __restrict__ slot_ids, float* __restrict__ coef,
    float* __restrict__ v_out) {
    const int t = blockIdx.x / heads, head = blockIdx.x % heads, lane = threadIdx.x;
    const int nk = kv_heads * dk, nv = heads * dv, C = 2 * nk + nv;
    const size_t cols = (size_t)C + nv + 2 * heads;
    const int r = tok_req[t];
    const int local = t - q_offsets[r];
    const float* tail = tails + (size_t)slot_ids[r] * (K - 1) * C;
    const int kv = head / (heads / kv_heads);
    float q[DELTA_PER_LANE], k[DELTA_PER_LANE], qq = 0.f, kk = 0.f;
#pragma unroll
    for (int e = 0; e < DELTA_PER_LANE; ++e) {
        const int i = lane + kWave * e;
        q[e] = k[e] = 0.f;
        if (i < dk) {
            q[e] = silu_f(conv_at<KT>(proj, cols, t, local, kv * dk + i, taps, K, tail, C));
            k[e] = silu_f(conv_at<KT>(proj, cols, t, local, nk + kv * dk + i, taps, K, tail, C));
        }
        qq = fmaf(q[e], q[e], qq);
        kk = fmaf(k[e], k[e], kk);
    }
    const float q_inv = 1.f / (sqrtf(wave_sum(qq) + unit_eps) * sqrtf((float)dk));
    const float k_inv = 1.f / sqrtf(wave_sum(kk) + unit_eps);
    const float* row = proj + (size_t)t * cols;
    const float beta = sigmoid(row[(size_t)C + nv + head]);
    const float g = expf(-expf(rate_log[head]) * softplus_f(row[(size_t)C + nv + heads + head] + rate_bias[head]));
    const size_t plane = (size_t)T * heads * dk;
#pragma unroll
    for (int e = 0; e < DELTA_PER_LANE; ++e) {
        const int i = lane + kWave * e;
        if (i >= dk) continue;
        const size_t at = ((size_t)t * heads + head) * dk + i;
        const float key = k[e] * k_inv;
        coef[at] = g;
        coef[plane + at] = g * key;
        coef[2 * plane + at] = beta * key;
        coef[3 * plane + at] = beta * key;
        coef[4 * plane + at] = q[e] * q_inv;
    }
    for (int i = lane; i < dv; i += kWave)
        v_out[((size_t)t * heads + head) * dv + i] =
            silu_f(conv_at<KT>(proj, cols, t, local, 2 * nk + head * dv + i, taps, K, tail, C));
}

// A thread per (request, channel): the new tail is the last K - 1 of (old tail, the step's inputs).
__global__ void conv_tail_update_kernel(const float* __restrict__ proj, int cols, float* __restrict__ tails, int C,
                                        int K, const int* __restrict__ q_offsets, const int* __restrict__ slot_ids) {
    const int r = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int first = q_offsets[r], n = q_offsets[r + 1] - first;
    float* tail = tails + (size_t)slot_ids[r] * (K - 1) * C;
    float keep[CONV_MAX_TAPS];
    for (int m = 0; m < K - 1; ++m) {
        const int at = n + m;               // place in (old tail, inputs)
        keep[m] = at < K - 1 ? tail[(size_t)at * C + c] : proj[(size_t)(first + at - (K - 1)) * cols + c];
    }
    for (int m = 0; m < K - 1; ++m) tail[(size_t)m * C + c] = keep[m];
}

constexpr int SCAN_LANES = 16;        // lanes that share a column's key rows: one DPP row

// Sum over the 16 lanes of a DPP row, every lane getting a total: neighbours, then pairs, then the
// quads by two rotations.  Lanes of different quads add the quads' sums in different orders, so
// their totals may differ in the last bit; which lane adds in which order is fixed, so a token's
// result is the same bits in every step that holds it.
__device__ __forceinline__ float lanes16_total(float v) {
    v += row_move<0xB1>(v);         // lane ^ 1
    v += row_move<0x4E>(v);         // lane ^ 2
    v += row_move<0x124>(v);        // the quad four lanes on
    v += row_move<0x128>(v);        // the two quads eight lanes on
    return v;
}

// ROWS floats from memory that is 16-byte aligned where ROWS is a multiple of four (the state's rows).
template <int ROWS>
__device__ __forceinline__ void load_rows(float (&dst)[ROWS], const float* __restrict__ p) {
    if constexpr (ROWS % 4 == 0) {
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
            const float4 q = *reinterpret_cast<const float4*>(p + r);
            dst[r] = q.x; dst[r + 1] = q.y; dst[r + 2] = q.z; dst[r + 3] = q.w;
        }
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) dst[r] = p[r];
    }
}

// Pointers into LDS, said to be so: through a plain pointer the compiler may fall back on flat
// loads, which wait on the memory counter too, and a wait for one of them then waits for every
// load of the next stage that is still on its way from memory.
typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) const void* glb_ptr_t;
typedef __attribute__((address_space(3))) float lds_f;
typedef __attribute__((address_space(3))) const float lds_cf;
typedef float float4_v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const float4_v lds_cf4;

template <int ROWS>
__device__ __forceinline__ void lds_rows(float (&dst)[ROWS], const float* generic) {
    lds_cf* p = (lds_cf*)generic;
    if constexpr (ROWS % 4 == 0) {
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
            const float4_v q = *(lds_cf4*)(p + r);
            dst[r] = q.x; dst[r + 1] = q.y; dst[r + 2] = q.z; dst[r + 3] = q.w;
        }
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) dst[r] = p[r];
    }
}

// What a lane needs of one token: its run of each of the vectors, and its column's value.  REMOVE: the
// recurrence has a removal term (five vectors: decay, probe, removal, write, read); else three (decay,
// write, read), and probe and removal are never touched.
template <int ROWS, bool REMOVE>
struct TokenRows {
    float decay[ROWS], probe[REMOVE ? ROWS : 1], removal[REMOVE ? ROWS : 1], write[ROWS], read_by[ROWS], value;
    // stage: the stage's vectors [5 or 3][CHUNK][DKP] (`plane` floats a vector, `dkp` a token), values: [CHUNK][columns]
    __device__ __forceinline__ void load(const float* stage, const float* values, int tt, int lane, int col, int plane,
                                         int dkp, int columns) {
        const float* at = stage + tt * dkp + lane * ROWS;
        if constexpr (REMOVE) {
            lds_rows<ROWS>(probe, at + plane);
            lds_rows<ROWS>(decay, at);
            lds_rows<ROWS>(removal, at + 2 * plane);
            lds_rows<ROWS>(write, at + 3 * plane);
            lds_rows<ROWS>(read_by, at + 4 * plane);
        } else {
            lds_rows<ROWS>(decay, at);
            lds_rows<ROWS>(write, at + plane);
            lds_rows<ROWS>(read_by, at + 2 * plane);
        }
        value = ((lds_cf*)values)[tt * columns + col];
    }
};

// grid (column blocks, heads, requests); a workgroup owns COLS value channels (16 lanes each).  A
// lane holds the ROWS key rows lane * ROWS ... of its column (16 ROWS >= dk); the tokens' vectors pass
// through LDS in stages of CHUNK tokens.  Where the key rows fill a stage's rows (dk = 16 ROWS) the
// stages are a ring that loads from memory fill directly, two stages ahead of the one being worked
// through (a stage's trip takes about 2 us, its eight tokens' work a little more); else the next stage
// travels through registers.  The state lies in memory as [slot, head, value, key]: a column's key
// rows in a row.  (Workgroups of four columns, one wave each, were measured too: 1,020 us against
// 594 for a 2,048-token request of 16 heads of 128 x 128.)
// DEEP: a token's vectors are read a token ahead (more registers, fewer waves a SIMD: for steps
// of long portions; steps of lone tokens are bound by the states' trip to memory and want the waves).
// REMOVE = false is the recurrence without its removal term, S <- diag(decay) S + write v^T, over three
// vectors a token: then only the state's own multiply-add ties a token to the next (no sum over the
// lanes stands before it), and the read-outs' sums of neighbouring tokens overlap.
template <int ROWS, int CHUNK, bool DEEP, int COLS, bool REMOVE>
__global__ __launch_bounds__(COLS * SCAN_LANES) void delta_scan_kernel(
    const float* __restrict__ coef, const float* __restrict__ v, float* __restrict__ state, float* __restrict__ out,
    const int* __restrict__ q_offsets, const int* __restrict__ slot_ids, int T, int heads, int dk, int dv) {
    constexpr int SCAN_COLUMNS = COLS, SCAN_THREADS = COLS * SCAN_LANES;
    constexpr int DKP = ROWS * SCAN_LANES;                 // key rows with padding
    constexpr int NP = REMOVE ? 5 : 3;                     // vectors a token
    constexpr int VEC = NP * CHUNK * DKP;                  // floats of a stage's vectors
    constexpr int PER_THREAD = VEC / SCAN_THREADS;
    static_assert(VEC % SCAN_THREADS == 0 && CHUNK * SCAN_COLUMNS <= SCAN_THREADS, "stage does not fit the threads");
    // stages in LDS: a ring of three for long portions, two for steps of lone tokens (less LDS, more
    // workgroups a CU); the loads that go through registers use two of them
    constexpr int NS = DEEP ? 3 : 2, AHEAD = NS - 1;
    __shared__ __attribute__((aligned(16))) float vec[NS][NP][CHUNK][DKP];
    // a stage's values [CHUNK][COLS], in a slot of whole 64-lane loads
    constexpr int VAL_SLOT = ((CHUNK * COLS + kWave - 1) / kWave) * kWave;
    __shared__ __attribute__((aligned(16))) float val[NS][VAL_SLOT];
    const int tid = threadIdx.x;
    const int col = tid / SCAN_LANES, lane = tid % SCAN_LANES;
    const int head = blockIdx.y, req = blockIdx.z;
    const int j = blockIdx.x * SCAN_COLUMNS + col;         // the value channel
    const int first = q_offsets[req], last = q_offsets[req + 1];
    float* S_home = state + (((size_t)slot_ids[req] * heads + head) * dv + (j < dv ? j : 0)) * dk + lane * ROWS;
    const bool whole = (dk % 4 == 0) && (ROWS % 4 == 0) && (lane + 1) * ROWS <= dk && j < dv;
    float S[ROWS];
    if (whole) {
        load_rows<ROWS>(S, S_home);
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) S[r] = (lane * ROWS + r < dk && j < dv) ? S_home[r] : 0.f;
    }
    const size_t plane = (size_t)T * heads * dk;
    float next_vec[PER_THREAD], next_val = 0.f;

    // a stage's numbers from memory into registers (zeros behind the request's end and behind dk)
    auto fetch = [&](int t0) {
        const int count = min(CHUNK, last - t0);
#pragma unroll
        for (int k = 0; k < PER_THREAD; ++k) {
            const int idx = tid + k * SCAN_THREADS;
            const int i = idx % DKP, tt = (idx / DKP) % CHUNK, c = idx / (DKP * CHUNK);
            next_vec[k] = (tt < count && i < dk) ? coef[c * plane + ((size_t)(t0 + tt) * heads + head) * dk + i] : 0.f;
        }
        if (tid < CHUNK * SCAN_COLUMNS) {
            const int cc = tid % SCAN_COLUMNS, tt = tid / SCAN_COLUMNS;
            const int jj = blockIdx.x * SCAN_COLUMNS + cc;
            next_val = (tt < count && jj < dv) ? v[((size_t)(t0 + tt) * heads + head) * dv + jj] : 0.f;
        }
    };
    auto park = [&](int buffer, bool vectors) {
        lds_f* flat = (lds_f*)&vec[buffer][0][0][0];
        if (vectors) {
#pragma unroll
            for (int k = 0; k < PER_THREAD; ++k) flat[tid + k * SCAN_THREADS] = next_vec[k];
        }
        if (tid < CHUNK * SCAN_COLUMNS) ((lds_f*)&val[buffer][0])[tid] = next_val;
    };
    // Where the key rows fill a stage's rows without padding (dk = 16 ROWS), the vectors go from memory
    // straight into LDS, 16 bytes a lane and 1 KB an instruction, past the registers: nothing of the
    // token loop waits for them.  A token behind the request's end is its last token once more.
    constexpr int DIRECT_LOADS = VEC / 256;
    constexpr bool CAN_DIRECT = VEC % 256 == 0;
    const bool direct = CAN_DIRECT && dk == DKP;
    auto fetch_direct = [&](int t0, int buffer) {
        const int wave = tid / kWave, lane64 = tid % kWave;
        for (int idx = wave; idx < DIRECT_LOADS; idx += SCAN_THREADS / kWave) {
            const int f = idx * 256 + lane64 * 4;
            const int i = f % DKP, tt = (f / DKP) % CHUNK, c = f / (DKP * CHUNK);
            const int t = min(t0 + tt, last - 1);
            const float* src = coef + c * plane + ((size_t)t * heads + head) * dk + i;
            __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(&vec[buffer][0][0][0] + idx * 256), 16, 0, 0);
        }
        // the values, four bytes a lane (a column behind dv reads the last one's: it is never written)
        for (int idx = wave; idx * kWave < CHUNK * SCAN_COLUMNS; idx += SCAN_THREADS / kWave) {
            const int f = idx * kWave + lane64;
            const int cc = f % SCAN_COLUMNS, tt = min(f / SCAN_COLUMNS, CHUNK - 1);
            const int jj = min(blockIdx.x * SCAN_COLUMNS + cc, dv - 1);
            const int t = min(t0 + tt, last - 1);
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(v + ((size_t)t * heads + head) * dv + jj),
                                             (lds_ptr_t)(&val[buffer][0] + idx * kWave), 4, 0, 0);
        }
    };

    // a stage's tokens, one after the other, from LDS stage `buffer`
    auto work = [&](int buffer, int t0, int count) {
        // a token's vectors are read from LDS while the token before it is worked through: only the
        // state itself ties one token to the next
        TokenRows<ROWS, REMOVE> rows[DEEP ? 2 : 1];
        if (DEEP) rows[0].load(&vec[buffer][0][0][0], &val[buffer][0], 0, lane, col, CHUNK * DKP, DKP, COLS);
        auto one = [&](int tt, const TokenRows<ROWS, REMOVE>& now) {
            float taken = 0.f, taken2 = 0.f;
            if constexpr (REMOVE) {
#pragma unroll
                for (int r = 0; r < ROWS; r += 2) {
                    taken = fmaf(now.probe[r], S[r], taken);
                    if (r + 1 < ROWS) taken2 = fmaf(now.probe[r + 1], S[r + 1], taken2);
                }
                taken = lanes16_total(taken + taken2);
            }
            float read = 0.f, read2 = 0.f;
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                float s = fmaf(now.write[r], now.value, now.decay[r] * S[r]);
                if constexpr (REMOVE) s = fmaf(-now.removal[r], taken, s);
                S[r] = s;
                if (r & 1) read2 = fmaf(s, now.read_by[r], read2);
                else read = fmaf(s, now.read_by[r], read);
            }
            read = lanes16_total(read + read2);
            if (lane == 0 && j < dv) out[((size_t)(t0 + tt) * heads + head) * dv + j] = read;
        };
        if (DEEP && count == CHUNK) {
#pragma unroll
            for (int tt = 0; tt < CHUNK; ++tt) {
                if (tt + 1 < CHUNK)
                    rows[DEEP ? (tt + 1) & 1 : 0].load(&vec[buffer][0][0][0], &val[buffer][0], tt + 1, lane, col,
                                                       CHUNK * DKP, DKP, COLS);
                one(tt, rows[DEEP ? tt & 1 : 0]);
            }
        } else {
            for (int tt = 0; tt < count; ++tt) {
                rows[0].load(&vec[buffer][0][0][0], &val[buffer][0], tt, lane, col, CHUNK * DKP, DKP, COLS);
                one(tt, rows[0]);
            }
        }
    };
    if (direct) {
        // the ring: AHEAD stages are on their way while one is worked through.  The memory counter
        // counts a wave's loads (and its stores of read-outs, which only makes the wait stricter) in
        // order: when at most the loads of the AHEAD - 1 youngest stages are left, the next stage is there.
        constexpr int PER_WAVE = DIRECT_LOADS / (SCAN_THREADS / kWave);
        constexpr int LEFT = (AHEAD - 1) * PER_WAVE < 63 ? (AHEAD - 1) * PER_WAVE : 63;
        for (int a = 0; a < AHEAD; ++a)
            if (first + a * CHUNK < last) fetch_direct(first + a * CHUNK, a);
        if (first + (AHEAD - 1) * CHUNK < last) wait_vmcnt<LEFT>();     // all AHEAD stages were asked for
        else wait_vmcnt<0>();
        __syncthreads();
        int buffer = 0;
        for (int t0 = first; t0 < last; t0 += CHUNK, buffer = buffer + 1 == NS ? 0 : buffer + 1) {
            if (t0 + AHEAD * CHUNK < last) fetch_direct(t0 + AHEAD * CHUNK, (buffer + AHEAD) % NS);
            work(buffer, t0, min(CHUNK, last - t0));
            // the youngest stages may still travel; none is asked for beyond the request's end
            if (t0 + AHEAD * CHUNK < last) wait_vmcnt<LEFT>();
            else wait_vmcnt<0>();
            __syncthreads();        // the next stage is there; this one has been read
        }
    } else {
        fetch(first);
        park(0, true);
        __syncthreads();
        int buffer = 0;
        for (int t0 = first; t0 < last; t0 += CHUNK, buffer ^= 1) {
            const bool more = t0 + CHUNK < last;
            if (more) fetch(t0 + CHUNK);
            work(buffer, t0, min(CHUNK, last - t0));
            if (more) park(buffer ^ 1, true);
            __syncthreads();        // the other stage is full; this one has been read
        }
    }
    if (whole) {
#pragma unroll
        for (int r = 0; r < ROWS; r += 4)
            *reinterpret_cast<float4*>(S_home + r) = make_float4(S[r], S[r + 1], S[r + 2], S[r + 3]);
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
            if (lane * ROWS + r < dk && j < dv) S_home[r] = S[r];
    }
}

}  // namespace lc

using namespace lc;

LC_API int lc_general_delta_prepare(const float* proj, int T, int heads, int dim, int inner, const float* decay_out,
                                    const float* decay_bias, const float* removal_bias, float unit_eps,
                                    float decay_scale, float* coef, float* v_out, hipStream_t stream) {
    LC_CHECK(T >= 0 && heads > 0 && dim > 0 && inner >= 0, "general_delta_prepare: bad sizes");
    LC_CHECK(dim <= DELTA_MAX_KEY, "general_delta_prepare: heads of %d key channels are above %d", dim, DELTA_MAX_KEY);
    LC_CHECK(inner <= DELTA_MAX_INNER, "general_delta_prepare: an inner size of %d is above %d", inner, DELTA_MAX_INNER);
    if (T == 0) return 0;
    LC_CHECK(proj && decay_bias && removal_bias && coef && v_out && (decay_out || inner == 0),
             "general_delta_prepare: null pointer");
    LC_CHECK((long long)T * heads < (1ll << 31), "general_delta_prepare: too many heads");
    general_delta_prepare_kernel<<<T * heads, kWave, 0, stream>>>(proj, T, heads, dim, inner, decay_out, decay_bias,
                                                                  removal_bias, unit_eps, decay_scale, coef, v_out);
    LC_LAUNCH_CHECK("general_delta_prepare");
    return 0;
}

LC_API int lc_gated_delta_prepare(const float* proj, int T, int heads, int kv_heads, int dk, int dv, int K,
                                  const float* taps, const float* tails, int tail_slots, const float* rate_log,
                                  const float* rate_bias, float unit_eps, const int* tok_req, const int* q_offsets,
                                  const int* slot_ids, float* coef, float* v_out, hipStream_t stream) {
    LC_CHECK(T >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dk > 0 && dv > 0,
             "gated_delta_prepare: bad sizes");
    LC_CHECK(dk <= DELTA_MAX_KEY, "gated_delta_prepare: heads of %d key channels are above %d", dk, DELTA_MAX_KEY);
    LC_CHECK(K >= 1 && K <= CONV_MAX_TAPS, "gated_delta_prepare: %d taps are outside 1..%d", K, CONV_MAX_TAPS);
    if (T == 0) return 0;
    LC_CHECK(proj && taps && rate_log && rate_bias && tok_req && q_offsets && slot_ids && coef && v_out &&
                 (tails || K == 1) && tail_slots >= 0,
             "gated_delta_prepare: null pointer");
    LC_CHECK((long long)T * heads < (1ll << 31), "gated_delta_prepare: too many heads");
#define LC_PREPARE(KT)                                                                                              \
    gated_delta_prepare_kernel<KT><<<T * heads, kWave, 0, stream>>>(proj, T, heads, kv_heads, dk, dv, K, taps, tails, \
                                                                    rate_log, rate_bias, unit_eps, tok_req, q_offsets, \
                                                                    slot_ids, coef, v_out)
    switch (K) {
        case 1: LC_PREPARE(1); break;
        case 2: LC_PREPARE(2); break;
        case 3: LC_PREPARE(3); break;
        case 4: LC_PREPARE(4); break;
        case 5: LC_PREPARE(5); break;
        case 6: LC_PREPARE(6); break;
        case 7: LC_PREPARE(7); break;
        case 8: LC_PREPARE(8); break;
        default: LC_PREPARE(0); break;
    }
#undef LC_PREPARE
    LC_LAUNCH_CHECK("gated_delta_prepare");
    return 0;
}

LC_API int lc_conv_tail_update(const float* proj, int cols, int T, float* tails, int tail_slots, int C, int K,
                               const int* q_offsets, const int* slot_ids, int R, hipStream_t stream) {
    LC_CHECK(T >= 0 && C > 0 && cols >= C && K >= 1 && K <= CONV_MAX_TAPS && R >= 0 && tail_slots >= 0,
             "conv_tail_update: bad sizes");
    if (R == 0 || K == 1) return 0;
    LC_CHECK(proj && tails && q_offsets && slot_ids, "conv_tail_update: null pointer");
    LC_CHECK(R <= 65535, "conv_tail_update: %d requests are above the grid's 65535", R);
    conv_tail_update_kernel<<<dim3((C + 255) / 256, R), 256, 0, stream>>>(proj, cols, tails, C, K, q_offsets, slot_ids);
    LC_LAUNCH_CHECK("conv_tail_update");
    return 0;
}

// coef [planes, T, heads dk]: five planes (decay, probe, removal, write, read) or three (decay, write,
// read: no removal term)
LC_API int lc_delta_scan(const float* coef, int planes, const float* v, float* state, int slots, float* out,
                         const int* q_offsets, const int* slot_ids, int R, int T, int heads, int dk, int dv,
                         hipStream_t stream) {
    LC_CHECK(R >= 0 && T >= 0 && heads > 0 && dk > 0 && dv > 0 && slots >= 0, "delta_scan: bad sizes");
    LC_CHECK(planes == 5 || planes == 3, "delta_scan: %d vectors a token are neither 5 nor 3", planes);
    LC_CHECK(dk <= DELTA_MAX_KEY, "delta_scan: heads of %d key channels are above %d", dk, DELTA_MAX_KEY);
    if (R == 0 || T == 0) return 0;
    LC_CHECK(coef && v && state && out && q_offsets && slot_ids, "delta_scan: null pointer");
    LC_CHECK(R <= 65535 && heads <= 65535, "delta_scan: too many requests or heads for the grid");
    const bool deep = T >= 16 * R;       // portions of prompts, mostly
    const dim3 grid((dv + 15) / 16, heads, R);
#define LC_SCAN_AS(ROWS, CHUNK, DEEP, COLS, REMOVE)                                                        \
    delta_scan_kernel<ROWS, CHUNK, DEEP, COLS, REMOVE><<<grid, COLS * SCAN_LANES, 0, stream>>>(              \
        coef, v, state, out, q_offsets, slot_ids, T, heads, dk, dv)
#define LC_SCAN(ROWS, CHUNK)                                            \
    do {                                                                \
        if (planes == 5) {                                              \
            if (deep) LC_SCAN_AS(ROWS, CHUNK, true, 16, true);          \
            else LC_SCAN_AS(ROWS, CHUNK, false, 16, true);              \
        } else {                                                        \
            if (deep) LC_SCAN_AS(ROWS, CHUNK, true, 16, false);         \
            else LC_SCAN_AS(ROWS, CHUNK, false, 16, false);             \
        }                                                               \
    } while (0)
    if (dk <= 16) LC_SCAN(1, 16);
    else if (dk <= 32) LC_SCAN(2, 16);
    else if (dk <= 64) LC_SCAN(4, 16);
    else if (dk <= 128) LC_SCAN(8, 8);
    else LC_SCAN(16, 4);
#undef LC_SCAN_AS
#undef LC_SCAN
    LC_LAUNCH_CHECK("delta_scan");
    return 0;
}
