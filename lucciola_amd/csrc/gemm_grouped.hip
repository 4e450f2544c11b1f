// Many small products in one launch: out_g = x_g . w_g^T for groups g, each with a matrix of
// its own, as true 32-bit products (operands widened to float32, v_mfma_f32_16x16x4_f32) with
// the arithmetic and the order of additions of gemm_generic.hip (K in chunks of 256, four k at
// a time within a chunk, the chunks' sums added from 0): an element's bits do not depend on how
// many rows or groups share the launch.
//
// Two ways to say which rows belong to which group:
//   heads    every group has the same M rows; group g reads its K columns of a wider x at column
//            g * x_group and writes its N columns of a wider out at column g * out_group (the
//            heads of an attention layer: a product per head over all tokens);
//   lists    the rows are sorted by group: group g owns rows row_start[g] .. row_start[g + 1] - 1
//            of out, and tile_start[g] counts the tiles of BM rows of the groups before it (both
//            made on the device: the experts of a routed feed-forward, whose counts the host
//            never sees).  Row m of x is gather[m] where a gather list is given.  The grid has
//            room for the most tiles there can be; a workgroup beyond the last tile leaves.
// The sums may pass an activation, or be multiplied by sigmoid(gate) read at the output's place
// in a tensor of gates, before they are stored.
#include "common.h"

#include "activations.h"

namespace lc {

constexpr int GG_N = 64, GG_K = 16, GG_CHUNK = 256, GG_PAD = 16;
typedef float floatx4 __attribute__((ext_vector_type(4)));

static thread_local int g_grouped_fast = 1;

struct GroupedArgs {
    const void* x; long long ldx, x_group;
    const void* w;
    void* out; long long ldo, out_group;
    int M, N, K, G;
    const int* gather; const int* row_start; const int* tile_start;
    int epilogue;
    const void* gate; long long ldg, gate_group;
};

template <typename TX, typename TW, typename TO, int BM, int WM, int WN>
__global__ __launch_bounds__(256, 2) void gemm_grouped_kernel(GroupedArgs a) {
    static_assert(WM * WN == 4, "four waves");
    constexpr int BN = GG_N;
    constexpr int TM = BM / 16 / WM, TN = BN / 16 / WN;
    constexpr int XL = (BM * 4 + 255) / 256, WL = (BN * 4 + 255) / 256;
    __shared__ float xs[2][GG_K][BM + GG_PAD];
    __shared__ float ws[2][GG_K][BN + GG_PAD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int N = a.N, K = a.K;
    int g, r0, r_end;
    if (a.row_start) {
        const int tile = blockIdx.y;
        if (tile >= a.tile_start[a.G]) return;
        int lo = 0, hi = a.G - 1;                 // the last group whose first tile is not after this one
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (a.tile_start[mid] <= tile) lo = mid; else hi = mid - 1;
        }
        g = lo;
        r0 = a.row_start[g] + (tile - a.tile_start[g]) * BM;
        r_end = a.row_start[g + 1];
    } else {
        g = blockIdx.z;
        r0 = blockIdx.y * BM;
        r_end = a.M;
    }
    const int n0 = blockIdx.x * BN;
    const TX* x = reinterpret_cast<const TX*>(a.x) + (size_t)g * a.x_group;
    const TW* w = reinterpret_cast<const TW*>(a.w) + (size_t)g * N * K;
    const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
    const int chunks = (K + GG_CHUNK - 1) / GG_CHUNK;

    const int lrow = tid / 4, lk = (tid % 4) * 4;
    const bool vec_x = (K & 3) == 0 && (a.ldx & 3) == 0 && (a.x_group & 3) == 0 && ((uintptr_t)a.x % 16 == 0);
    const bool vec_w = (K & 3) == 0 && ((uintptr_t)a.w % 16 == 0);
    const TX* xrow[XL];
    const TW* wrow[WL];
    bool xlive[XL], wlive[WL];
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        const int row = lrow + 64 * u;
        xlive[u] = row < BM && r0 + row < r_end;
        const int m = xlive[u] ? r0 + row : r0;           // r0 < r_end: a tile has at least one row
        const long long src = a.gather ? a.gather[m] : m;
        xrow[u] = x + src * a.ldx + lk;
    }
#pragma unroll
    for (int u = 0; u < WL; ++u) {
        const int row = lrow + 64 * u;
        wlive[u] = row < BN && n0 + row < N;
        wrow[u] = w + (size_t)(wlive[u] ? n0 + row : 0) * K + lk;
    }
    float xr[XL][4], wr[WL][4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int u = 0; u < XL; ++u) {
            if (vec_x && k0 + lk + 3 < K) {
                load4(xr[u], xrow[u] + k0);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) xr[u][j] = k0 + lk + j < K ? to_f32(xrow[u][k0 + j]) : 0.f;
            }
            if (!xlive[u]) { xr[u][0] = xr[u][1] = xr[u][2] = xr[u][3] = 0.f; }
        }
#pragma unroll
        for (int u = 0; u < WL; ++u) {
            if (vec_w && k0 + lk + 3 < K) {
                load4(wr[u], wrow[u] + k0);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) wr[u][j] = k0 + lk + j < K ? to_f32(wrow[u][k0 + j]) : 0.f;
            }
            if (!wlive[u]) { wr[u][0] = wr[u][1] = wr[u][2] = wr[u][3] = 0.f; }
        }
    };
    auto put = [&](int stage) {
#pragma unroll
        for (int u = 0; u < XL; ++u)
            if (lrow + 64 * u < BM)
#pragma unroll
                for (int j = 0; j < 4; ++j) xs[stage][lk + j][lrow + 64 * u] = xr[u][j];
#pragma unroll
        for (int u = 0; u < WL; ++u)
            if (lrow + 64 * u < BN)
#pragma unroll
                for (int j = 0; j < 4; ++j) ws[stage][lk + j][lrow + 64 * u] = wr[u][j];
    };

    floatx4 total[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) total[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    int stage = 0;
    fetch(0);
    put(0);
    for (int c = 0; c < chunks; ++c) {
        floatx4 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
        const int k_end = min(K, (c + 1) * GG_CHUNK);
        for (int k0 = c * GG_CHUNK; k0 < k_end; k0 += GG_K) {
            __syncthreads();
            const int next = k0 + GG_K;
            const bool more = next < K;
            if (more) fetch(next);
            float av[4][TM], bv[4][TN];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int i = 0; i < TM; ++i) av[q][i] = xs[stage][4 * q + (lane >> 4)][wm + 16 * i + (lane & 15)];
#pragma unroll
                for (int j = 0; j < TN; ++j) bv[q][j] = ws[stage][4 * q + (lane >> 4)][wn + 16 * j + (lane & 15)];
            }
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[q][i], bv[q][j], acc[i][j], 0, 0, 0);
            stage ^= 1;
            if (more) put(stage);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) total[i][j][r] = __fadd_rn(total[i][j][r], acc[i][j][r]);
    }
    // lane l holds the rows 4 (l / 16) + r and the column l % 16 of each of its tiles
    TO* out = reinterpret_cast<TO*>(a.out) + (size_t)g * a.out_group;
    const TX* gate = a.gate ? reinterpret_cast<const TX*>(a.gate) + (size_t)g * a.gate_group : nullptr;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = r0 + wm + 16 * i + 4 * (lane >> 4) + r, n = n0 + wn + 16 * j + (lane & 15);
                if (m < r_end && n < N) {
                    float v = total[i][j][r];
                    if (a.epilogue == ACT_SIGMOID_GATE) v *= sigmoid(to_f32(gate[(size_t)m * a.ldg + n]));
                    else if (a.epilogue == ACT_SIGMOID_GROUP_GATE) v *= sigmoid(to_f32(gate[(size_t)m * a.ldg]));
                    else v = activate(v, a.epilogue);
                    out[(size_t)m * a.ldo + n] = from_f32<TO>(v);
                }
            }
}


// The same products for bfloat16 operands on v_mfma_f32_16x16x32_bf16 (float32 sums over all of K
// in order): steps of 32 k, both tiles in LDS as rows of 32 k (padded to 40: every operand is one
// conflict-free 16-byte read), the next step's pieces in registers while this one is multiplied.
// Rows and groups as above; K, the rows' strides and the groups' offsets must be multiples of 8.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
constexpr int GH_K = 32, GH_STRIDE = GH_K + 8;

template <typename TO, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(256, 2) void gemm_grouped_bf16_kernel(GroupedArgs a) {
    static_assert(WM * WN == 4, "four waves");
    constexpr int TM = BM / 16 / WM, TN = BN / 16 / WN;
    constexpr int XL = (BM * 4 + 255) / 256, WL = (BN * 4 + 255) / 256;   // 16-byte pieces a thread brings a step
    __shared__ __align__(16) bf16 xs[2][BM][GH_STRIDE];
    __shared__ __align__(16) bf16 ws[2][BN][GH_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 15, g = lane >> 4;
    const int N = a.N, K = a.K;
    int grp, r0, r_end;
    if (a.row_start) {
        const int tile = blockIdx.y;
        if (tile >= a.tile_start[a.G]) return;
        int lo = 0, hi = a.G - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (a.tile_start[mid] <= tile) lo = mid; else hi = mid - 1;
        }
        grp = lo;
        r0 = a.row_start[grp] + (tile - a.tile_start[grp]) * BM;
        r_end = a.row_start[grp + 1];
    } else {
        grp = blockIdx.z;
        r0 = blockIdx.y * BM;
        r_end = a.M;
    }
    const int n0 = blockIdx.x * BN;
    const bf16* x = reinterpret_cast<const bf16*>(a.x) + (size_t)grp * a.x_group;
    const bf16* w = reinterpret_cast<const bf16*>(a.w) + (size_t)grp * N * K;
    const int wm = (wave / WN) * (BM / WM), wn = (wave % WN) * (BN / WN);
    // loader: a thread brings 16-byte pieces (8 k) of rows of x and of w, 64 rows apart
    const int lrow = tid >> 2, lk = (tid & 3) * 8;
    bool xlive[XL], wlive[WL];
    const bf16* xrow[XL];
    const bf16* wrow[WL];
#pragma unroll
    for (int u = 0; u < XL; ++u) {
        const int row = lrow + 64 * u;
        xlive[u] = row < BM && r0 + row < r_end;
        const int m_src = xlive[u] ? r0 + row : r0;
        xrow[u] = x + (size_t)(a.gather ? a.gather[m_src] : m_src) * a.ldx + lk;
    }
#pragma unroll
    for (int u = 0; u < WL; ++u) {
        const int row = lrow + 64 * u;
        wlive[u] = row < BN && n0 + row < N;
        wrow[u] = w + (size_t)(wlive[u] ? n0 + row : 0) * K + lk;
    }
    bf16x8 zero;
#pragma unroll
    for (int i = 0; i < 8; ++i) zero[i] = static_cast<bf16>(0.f);
    bf16x8 xr[XL], wr[WL];
    auto fetch = [&](int k0) {
        const bool in = k0 + lk < K;                // K % 8 == 0: a piece is whole or absent
#pragma unroll
        for (int u = 0; u < XL; ++u) xr[u] = (xlive[u] && in) ? *reinterpret_cast<const bf16x8*>(xrow[u] + k0) : zero;
#pragma unroll
        for (int u = 0; u < WL; ++u) wr[u] = (wlive[u] && in) ? *reinterpret_cast<const bf16x8*>(wrow[u] + k0) : zero;
    };
    auto put = [&](int stage) {
#pragma unroll
        for (int u = 0; u < XL; ++u)
            if (lrow + 64 * u < BM) *reinterpret_cast<bf16x8*>(&xs[stage][lrow + 64 * u][lk]) = xr[u];
#pragma unroll
        for (int u = 0; u < WL; ++u)
            if (lrow + 64 * u < BN) *reinterpret_cast<bf16x8*>(&ws[stage][lrow + 64 * u][lk]) = wr[u];
    };
    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
    int stage = 0;
    fetch(0);
    put(0);
    for (int k0 = 0; k0 < K; k0 += GH_K) {
        __syncthreads();
        const bool more = k0 + GH_K < K;
        if (more) fetch(k0 + GH_K);
        bf16x8 av[TM], bv[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) av[i] = *reinterpret_cast<const bf16x8*>(&xs[stage][wm + 16 * i + col][8 * g]);
#pragma unroll
        for (int j = 0; j < TN; ++j) bv[j] = *reinterpret_cast<const bf16x8*>(&ws[stage][wn + 16 * j + col][8 * g]);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av[i], bv[j], acc[i][j], 0, 0, 0);
        stage ^= 1;
        if (more) put(stage);
    }
    // C = x . w^T with x as the first operand: the lane holds the rows 4 g + r, column col of a tile
    TO* out = reinterpret_cast<TO*>(a.out) + (size_t)grp * a.out_group;
    const bf16* gate = a.gate ? reinterpret_cast<const bf16*>(a.gate) + (size_t)grp * a.gate_group : nullptr;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = r0 + wm + 16 * i + 4 * g + r, n = n0 + wn + 16 * j + col;
                if (m < r_end && n < N) {
                    float v = acc[i][j][r];
                    if (a.epilogue == ACT_SIGMOID_GATE) v *= sigmoid(to_f32(gate[(size_t)m * a.ldg + n]));
                    else if (a.epilogue == ACT_SIGMOID_GROUP_GATE) v *= sigmoid(to_f32(gate[(size_t)m * a.ldg]));
                    else v = activate(v, a.epilogue);
                    out[(size_t)m * a.ldo + n] = from_f32<TO>(v);
                }
            }
}

template <typename TO>
static int launch_grouped_bf16(const GroupedArgs& a, int max_tiles, int tile_rows, hipStream_t stream) {
    if (tile_rows == 16) {
        dim3 grid((a.N + 63) / 64, a.row_start ? max_tiles : (a.M + 15) / 16, a.row_start ? 1 : a.G);
        gemm_grouped_bf16_kernel<TO, 16, 64, 1, 4><<<grid, 256, 0, stream>>>(a);
    } else if (tile_rows == 128) {
        dim3 grid((a.N + 127) / 128, a.row_start ? max_tiles : (a.M + 127) / 128, a.row_start ? 1 : a.G);
        gemm_grouped_bf16_kernel<TO, 128, 128, 2, 2><<<grid, 256, 0, stream>>>(a);
    } else {
        dim3 grid((a.N + 63) / 64, a.row_start ? max_tiles : (a.M + 63) / 64, a.row_start ? 1 : a.G);
        gemm_grouped_bf16_kernel<TO, 64, 64, 2, 2><<<grid, 256, 0, stream>>>(a);
    }
    LC_LAUNCH_CHECK("gemm_grouped_bf16");
    return 0;
}

template <typename TX, typename TW, typename TO>
static int launch_grouped(const GroupedArgs& a, int max_tiles, int tile_rows, hipStream_t stream) {
    const int nb = (a.N + GG_N - 1) / GG_N;
    if (tile_rows == 16) {
        dim3 grid(nb, a.row_start ? max_tiles : (a.M + 15) / 16, a.row_start ? 1 : a.G);
        gemm_grouped_kernel<TX, TW, TO, 16, 1, 4><<<grid, 256, 0, stream>>>(a);
    } else {
        dim3 grid(nb, a.row_start ? max_tiles : (a.M + 63) / 64, a.row_start ? 1 : a.G);
        gemm_grouped_kernel<TX, TW, TO, 64, 2, 2><<<grid, 256, 0, stream>>>(a);
    }
    LC_LAUNCH_CHECK("gemm_grouped");
    return 0;
}

}  // namespace lc

using namespace lc;

// Tests and tuning: whether bfloat16 operands may take the bfloat16 matrix instruction (1, the default)
// or always the true 32-bit product (0), for the calling thread.  Returns the setting before.
LC_API int lc_gemm_grouped_fast(int on) {
    const int before = g_grouped_fast;
    if (on >= 0) g_grouped_fast = on ? 1 : 0;
    return before;
}

// Whether tiles of `tile_rows` rows exist for these operand types (16 and 64: always; 128: the
// bfloat16 kernel only).  The lists' tile_start must have been made for the size that is asked for.
LC_API int lc_gemm_grouped_takes_tile(int tile_rows, int x_dt, int w_dt) {
    if (tile_rows == 16 || tile_rows == 64) return 1;
    return tile_rows == 128 && x_dt == DT_BF16 && w_dt == DT_BF16 && g_grouped_fast ? 1 : 0;
}

// x, gate: dtype x_dt; w: w_dt; out: out_dt.  lists: row_start and tile_start [G + 1] on the
// device, max_tiles the grid's room; M then is the number of sorted rows.  heads: both null.
LC_API int lc_gemm_grouped(const void* x, int x_dt, long long ldx, long long x_group, const void* w, int w_dt,
                           void* out, int out_dt, long long ldo, long long out_group, int M, int N, int K, int G,
                           const int* gather, const int* row_start, const int* tile_start, int max_tiles,
                           int tile_rows, int epilogue, const void* gate, long long ldg, long long gate_group,
                           hipStream_t stream) {
    LC_CHECK(M >= 0 && N > 0 && K > 0 && G > 0, "grouped product: bad sizes M=%d N=%d K=%d G=%d", M, N, K, G);
    if (M == 0) return 0;
    LC_CHECK(x && w && out, "grouped product: null pointer");
    LC_CHECK((row_start == nullptr) == (tile_start == nullptr), "grouped product: the lists come together");
    LC_CHECK(row_start || gather == nullptr, "grouped product: a gather list needs the rows' lists");
    LC_CHECK(!row_start || max_tiles > 0, "grouped product: no room for tiles");
    LC_CHECK(epilogue >= ACT_NONE && epilogue <= ACT_SIGMOID_GROUP_GATE, "grouped product: unknown epilogue %d", epilogue);
    LC_CHECK((epilogue != ACT_SIGMOID_GATE && epilogue != ACT_SIGMOID_GROUP_GATE) || gate, "grouped product: no gates");
    LC_CHECK(tile_rows == 16 || tile_rows == 64 || tile_rows == 128, "grouped product: tiles of %d rows", tile_rows);
    LC_CHECK(G <= 65535 && (row_start ? max_tiles : (M + 15) / 16) <= 65535, "grouped product: too many tiles");
    GroupedArgs a{x, ldx, x_group, w, out, ldo, out_group, M, N, K, G, gather, row_start, tile_start,
                  epilogue, gate, ldg, gate_group};
    // bfloat16 operands whose pieces of 8 are whole and aligned: the bfloat16 matrix instruction
    if (x_dt == DT_BF16 && w_dt == DT_BF16 && K % 8 == 0 && ldx % 8 == 0 && x_group % 8 == 0 &&
        (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && g_grouped_fast) {
        if (out_dt == DT_BF16) return launch_grouped_bf16<bf16>(a, max_tiles, tile_rows, stream);
        if (out_dt == DT_F32) return launch_grouped_bf16<float>(a, max_tiles, tile_rows, stream);
    }
    LC_CHECK(tile_rows != 128 || !row_start, "grouped product: lists made for tiles of 128 rows need whole aligned bfloat16 pieces");
    if (tile_rows == 128) tile_rows = 64;
    const int key = x_dt * 4 + w_dt * 2 + out_dt;
    switch (key) {
        case 0: return launch_grouped<float, float, float>(a, max_tiles, tile_rows, stream);
        case 2: return launch_grouped<float, bf16, float>(a, max_tiles, tile_rows, stream);
        case 4: return launch_grouped<bf16, float, float>(a, max_tiles, tile_rows, stream);
        case 5: return launch_grouped<bf16, float, bf16>(a, max_tiles, tile_rows, stream);
        case 6: return launch_grouped<bf16, bf16, float>(a, max_tiles, tile_rows, stream);
        case 7: return launch_grouped<bf16, bf16, bf16>(a, max_tiles, tile_rows, stream);
        default:
            LC_CHECK(false, "grouped product: unsupported dtypes x=%d w=%d out=%d", x_dt, w_dt, out_dt);
    }
    return 0;
}
