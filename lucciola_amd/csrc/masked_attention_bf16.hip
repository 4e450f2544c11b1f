// The masked attention of masked_attention.hip on the matrix cores, for bfloat16 caches whose sizes fit:
// key heads of a multiple of 8 entries up to 128, value heads of a multiple of 16 up to 128, pages of a
// multiple of 16 tokens.  Same formulas, same cache (keys token-major, values transposed inside a page);
// scores, softmax, sink, bias and the heads' combination are float32, the two products take bfloat16
// operands: the weights go into P.V as two bfloat16 numbers each (the rounded weight and the rounding's
// remainder, two products), so that they count with 16 bits of mantissa and not with 8.
//
// Work comes as the step's tiles (first token row, tokens, request, first position: up to 16 tokens of one
// request); a workgroup of eight waves serves a tile and one kv head.
//   A tile of several tokens: a wave's 16 columns are the tile's tokens for one query head of the kv head's
//   group; where the group has fewer than eight heads, the waves of a head share out the blocks of keys.
//   A lone token: the 16 columns are query heads of the group, and all eight waves share out the blocks.
// Waves that shared a column's keys leave their maxima, sums and rows in LDS, and the first of them takes the
// others in, in their order.  A wave asks for the next block's keys before it works on this one's.
// In a step of lone tokens only, with fewer workgroups than the card has room for, a token's blocks are also
// shared out over several workgroups (the grid's last place); each leaves its joined sums in a workspace, and a
// second kernel takes them in, in their order, and finishes the columns.
// Keys are walked in blocks of 16 (one part of a page).  S^T = K Q^T (16x16x32: a lane's operand is 16 bytes
// in a row of a key, straight from memory) leaves a lane with four keys of one query column, which is the
// operand P^T of O^T += V^T P^T (16x16x16; V^T's operand is four neighbouring keys of one value entry, 8
// bytes in a row of the transposed page), so the weights never leave the registers.
#include "common.h"

namespace lc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int MB_WAVES = 8;
constexpr int MB_THREADS = MB_WAVES * kWave;

struct MaskedArgs {
    const bf16* q;
    const bf16* k_cache;
    const bf16* v_cache;
    const int* tiles;
    const int* block_table;
    int max_blocks, page_size, heads, kv_heads, d, dv;
    float scale;
    int chunk, window;
    const float* r1;
    const float* r2;
    const float* sink;
    float lambda;
    int unit_out;
    float eps, out_scale;
    const float* gate;
    int gate_stride, gate_column;
    bf16* out;
    float* shares;      // where a lone token's keys are shared out over workgroups: their sums, joined by a second kernel
    int zsplits;
    int lone_only;      // the tiles of several tokens are another kernel's
    int wave_blocks;    // blocks of a stage for every wave that shares a head's keys, in the kernel that stages them
};

// floats a wave leaves per lane and map where key ranges are joined: maximum, sum, the lane's part of O^T
template <int DVB> constexpr int share_floats() { return DVB * 4 + 2; }

__device__ __forceinline__ short bits_of(__bf16 v) { return __builtin_bit_cast(short, v); }

// over the four lanes that hold one query column (lane, lane ^ 16, lane ^ 32, lane ^ 48)
__device__ __forceinline__ float column_max4(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, kWave));
    return fmaxf(v, __shfl_xor(v, 32, kWave));
}
__device__ __forceinline__ float column_sum4(float v) {
    v += __shfl_xor(v, 16, kWave);
    return v + __shfl_xor(v, 32, kWave);
}

template <int DVB, int MAPS>
struct ColumnState {
    float m[MAPS], l[MAPS];     // the column's reference point (the same in its four lanes); the lane's own part of the sum
    floatx4 o[MAPS][DVB];       // O^T: value entries 16 t + 4 (lane / 16) + i of the lane's query column
};

// One block of 16 keys for the lane's column: scores from the keys' and the queries' operands, mask, bias, the
// reference point and the sum, and the weighted values taken into O^T.
template <int DSTEPS, int DVB, int MAPS>
__device__ __forceinline__ void block_step(ColumnState<DVB, MAPS>& st, const MaskedArgs& a,
                                           const bf16x8 (&bq)[MAPS][DSTEPS], const bf16x8 (&ka)[MAPS][DSTEPS],
                                           const short4v (&va)[DVB], int key0, int pos, int lo, float bias1, float bias2,
                                           bool all_seen, int lane) {
    const int quad = lane >> 4;
    const int j0 = key0 + quad * 4;
    float far[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) far[v] = a.r1 ? bias1 * __logf(1.f + bias2 * (float)max(pos - (j0 + v), 0)) : 0.f;
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
        floatx4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < DSTEPS; ++i) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[m][i], bq[m][i], s, 0, 0, 0);
        float mx = -INFINITY;
        if (all_seen) {             // every column of the wave sees the whole block: nothing to mask
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                s[v] = fmaf(s[v], a.scale, -far[v]);
                mx = fmaxf(mx, s[v]);
            }
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int j = j0 + v;
                s[v] = (j >= lo && j <= pos) ? fmaf(s[v], a.scale, -far[v]) : -INFINITY;
                mx = fmaxf(mx, s[v]);
            }
        }
        // The column's reference point st.m moves only when a score outgrows it by e^8 (or it has none yet): until
        // then no lane asks its column's other three, the weights are exp(s - reference) <= e^8, and a lane keeps
        // its own part of the column's sum, which is added up when the column is finished.
        if (__any(mx > st.m[m] + 8.f)) {
            const float top = column_max4(mx);
            const float m_new = top > st.m[m] + 8.f ? top : st.m[m];
            const float alpha = m_new == st.m[m] ? 1.f : __expf(st.m[m] - m_new);       // 0 from no reference at all
            st.l[m] *= alpha;
#pragma unroll
            for (int t = 0; t < DVB; ++t) st.o[m][t] *= alpha;
            st.m[m] = m_new;
        }
        const float base = st.m[m] == -INFINITY ? 0.f : st.m[m];      // a column that has seen no key yet
        // A weight p >= 0 as two bfloat16 numbers: its upper 16 bits, and the upper 16 bits of what they leave
        // (p minus them is exact in float32): together p to 2^-15 of itself.
        float psum = 0.f;
        unsigned hi_bits[4], lw_bits[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float p = __expf(s[v] - base);
            psum += p;
            const unsigned whole = __float_as_uint(p), upper = whole & 0xffff0000u;
            hi_bits[v] = whole >> 16;
            lw_bits[v] = __float_as_uint(p - __uint_as_float(upper)) >> 16;
        }
        typedef unsigned uint2v __attribute__((ext_vector_type(2)));
        const short4v hi = __builtin_bit_cast(short4v, uint2v{hi_bits[0] | (hi_bits[1] << 16), hi_bits[2] | (hi_bits[3] << 16)});
        const short4v lw = __builtin_bit_cast(short4v, uint2v{lw_bits[0] | (lw_bits[1] << 16), lw_bits[2] | (lw_bits[3] << 16)});
        st.l[m] += psum;
        // the weights' upper halves into every block of value entries first, then the remainders: no product waits
        // for the one before it
#pragma unroll
        for (int t = 0; t < DVB; ++t) st.o[m][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(va[t], hi, st.o[m][t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < DVB; ++t) st.o[m][t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(va[t], lw, st.o[m][t], 0, 0, 0);
    }
}

template <int DSTEPS, int MAPS>
__device__ __forceinline__ void load_queries(bf16x8 (&bq)[MAPS][DSTEPS], const MaskedArgs& a, int tok, int head, int pos,
                                             int lane) {
    const int quad = lane >> 4;
#pragma unroll
    for (int m = 0; m < MAPS; ++m)
#pragma unroll
        for (int s = 0; s < DSTEPS; ++s) {
            const int e = s * 32 + quad * 8;
#pragma unroll
            for (int x = 0; x < 8; ++x) bq[m][s][x] = (__bf16)0.f;
            if (pos >= 0 && e < a.d)
                bq[m][s] = *reinterpret_cast<const bf16x8*>(a.q + ((size_t)tok * a.heads + head) * MAPS * a.d + m * a.d + e);
        }
}

template <int DVB, int MAPS>
__device__ __forceinline__ void clear_state(ColumnState<DVB, MAPS>& st) {
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
        st.m[m] = -INFINITY;
        st.l[m] = 0.f;
#pragma unroll
        for (int t = 0; t < DVB; ++t) st.o[m][t] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
}

// The lane's column: token row `tok`, head `head`, position `pos` (-1: no such column), first visible key `lo`.
// Blocks first, first + stride, ... <= last of 16 keys each.  Keys seen_from .. seen_to are seen by every column of
// the tile (a block inside them needs no mask).
template <int DSTEPS, int DVB, int MAPS>
__device__ __forceinline__ void attend_blocks(ColumnState<DVB, MAPS>& st, const MaskedArgs& a, int g, int tok, int head,
                                              int pos, int lo, const int* __restrict__ table, int first, int last,
                                              int stride, int seen_from, int seen_to, int lane) {
    const int quad = lane >> 4, col = lane & 15;
    const size_t k_row = (size_t)a.kv_heads * MAPS * a.d;
    bf16x8 bq[MAPS][DSTEPS];
    load_queries<DSTEPS, MAPS>(bq, a, tok, head, pos, lane);
    const float bias1 = (a.r1 && pos >= 0) ? a.r1[head] : 0.f, bias2 = (a.r1 && pos >= 0) ? a.r2[head] : 0.f;
    clear_state<DVB, MAPS>(st);
    auto load_keys = [&](bf16x8 (&dst)[MAPS][DSTEPS], int b) {
        const int key0 = b * 16;
        const size_t row0 = (size_t)table[key0 / a.page_size] * a.page_size + key0 % a.page_size;
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
#pragma unroll
            for (int s = 0; s < DSTEPS; ++s) {
                const int e = s * 32 + quad * 8;
#pragma unroll
                for (int x = 0; x < 8; ++x) dst[m][s][x] = (__bf16)0.f;
                if (e < a.d)
                    dst[m][s] = *reinterpret_cast<const bf16x8*>(a.k_cache + (row0 + col) * k_row + ((size_t)g * MAPS + m) * a.d + e);
            }
    };
    auto load_values = [&](short4v (&dst)[DVB], int b) {
        const int key0 = b * 16;
        const int page = table[key0 / a.page_size], within = key0 % a.page_size;
#pragma unroll
        for (int t = 0; t < DVB; ++t) {
            dst[t] = short4v{0, 0, 0, 0};
            if (t * 16 < a.dv)
                dst[t] = *reinterpret_cast<const short4v*>(
                    a.v_cache + ((size_t)page * a.kv_heads * a.dv + (size_t)g * a.dv + t * 16 + col) * a.page_size + within + quad * 4);
        }
    };
    // the next block's values travel ahead as well where the registers hold them
    constexpr bool VALUES_AHEAD = DSTEPS * MAPS * 4 + DVB * MAPS * 4 + DVB * 4 <= 120;
    bf16x8 ka[MAPS][DSTEPS], kn[MAPS][DSTEPS];
    short4v va[DVB], vn[DVB];
    if (first <= last) {
        load_keys(ka, first);
        if constexpr (VALUES_AHEAD) load_values(va, first);
    }
    for (int b = first; b <= last; b += stride) {
        const int key0 = b * 16;
        if constexpr (!VALUES_AHEAD) load_values(va, b);
        if (b + stride <= last) {           // on their way while this block is worked on
            load_keys(kn, b + stride);
            if constexpr (VALUES_AHEAD) load_values(vn, b + stride);
        }
        block_step<DSTEPS, DVB, MAPS>(st, a, bq, ka, va, key0, pos, lo, bias1, bias2,
                                      key0 >= seen_from && key0 + 15 <= seen_to, lane);
#pragma unroll
        for (int m = 0; m < MAPS; ++m)
#pragma unroll
            for (int i = 0; i < DSTEPS; ++i) ka[m][i] = kn[m][i];
        if constexpr (VALUES_AHEAD)
#pragma unroll
            for (int t = 0; t < DVB; ++t) va[t] = vn[t];
    }
}

// The lane's column is done: sink, the maps' combination, the unit norm, the gate; four entries a block written.
template <int DVB, int MAPS>
__device__ __forceinline__ void finish_column(const ColumnState<DVB, MAPS>& st, const MaskedArgs& a, int tok, int head,
                                              int pos, int lane) {
    const int quad = lane >> 4;
    floatx4 o[DVB];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
        float top = st.m[m], sunk = 0.f;
        if (a.sink && pos >= 0) {
            top = fmaxf(st.m[m], a.sink[head]);
            sunk = expf(a.sink[head] - top);
        }
        const float shrink = pos >= 0 ? expf(st.m[m] - top) : 0.f;
        const float denom = fmaf(column_sum4(st.l[m]), shrink, sunk);        // the four lanes' parts of the column's sum
        const float w = denom > 0.f ? shrink / denom : 0.f;
#pragma unroll
        for (int t = 0; t < DVB; ++t) {
            if (m == 0) o[t] = st.o[0][t] * w;
            else o[t] -= st.o[m][t] * (w * a.lambda);
        }
    }
    if (a.unit_out) {
        float ss = 0.f;
#pragma unroll
        for (int t = 0; t < DVB; ++t)
            if (t * 16 < a.dv)
#pragma unroll
                for (int i = 0; i < 4; ++i) ss = fmaf(o[t][i], o[t][i], ss);
        const float inv = a.out_scale / sqrtf(column_sum4(ss) / (float)a.dv + a.eps);
#pragma unroll
        for (int t = 0; t < DVB; ++t) o[t] *= inv;
    }
    if (pos < 0) return;
#pragma unroll
    for (int t = 0; t < DVB; ++t) {
        if (t * 16 >= a.dv) continue;
        const int e = t * 16 + quad * 4;
        short4v packed;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = o[t][i];
            if (a.gate) v = v / (1.f + expf(-a.gate[(size_t)tok * a.gate_stride + a.gate_column + (size_t)head * a.dv + e + i]));
            packed[i] = bits_of((__bf16)v);
        }
        *reinterpret_cast<short4v*>(a.out + ((size_t)tok * a.heads + head) * a.dv + e) = packed;
    }
}

template <int DSTEPS, int DVB, int MAPS>
__global__ __launch_bounds__(MB_THREADS) void masked_attention_bf16_kernel(MaskedArgs a) {
    __shared__ float meet[MB_WAVES - 1][kWave][DVB * 4 + 2];
    const int* tile = a.tiles + 4 * blockIdx.x;
    const int t0 = tile[0], n = tile[1], r = tile[2], p0 = tile[3];
    const int g = blockIdx.y, group = a.heads / a.kv_heads;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), col = lane & 15;
    const int* table = a.block_table + (size_t)r * a.max_blocks;
    auto first_key = [&](int p) {
        int lo = 0;
        if (a.chunk > 0) lo = p - p % a.chunk;
        if (a.window > 0) lo = max(lo, p - a.window + 1);
        return lo;
    };
    const bool lone = n == 1;
    const int z = blockIdx.z, zsplits = lone ? a.zsplits : 1;
    if (!lone && (z > 0 || a.lone_only)) return;
    // head places of a pass (a power of two up to the waves), and the waves that share a place's keys
    int places = 1;
    if (!lone)
        while (places < group && places < MB_WAVES) places *= 2;
    const int splits = MB_WAVES / places;
    const int place = wave % places, split = wave / places;
    // the blocks from the first token's first key to the last token
    const int first = first_key(p0) / 16, last = (p0 + n - 1) / 16;
    // what every token of the tile sees: from the last token's first key to the first token (a column without a token
    // or head computes on zeros there and is never written)
    const int seen_from = first_key(p0 + n - 1), seen_to = p0;
    const int heads_a_pass = lone ? 16 : places;
    ColumnState<DVB, MAPS> st;
    for (int h0 = 0; h0 < group; h0 += heads_a_pass) {
        // the lane's column: a token of the tile for the wave's head, or a head of the group for the lone token
        const int hh = lone ? h0 + col : h0 + place;
        const bool on = hh < group && (lone || col < n);
        const int head = g * group + (hh < group ? hh : 0);
        const int tok = lone ? t0 : t0 + (col < n ? col : 0);
        const int pos = on ? (lone ? p0 : p0 + col) : -1;
        const int lo = on ? first_key(pos) : 0;
        const bool wave_on = lone || h0 + place < group;
        if (wave_on)
            attend_blocks<DSTEPS, DVB, MAPS>(st, a, g, tok, head, pos, lo, table, first + z * splits + split, last,
                                             splits * zsplits, seen_from, seen_to, lane);
        if (splits > 1) {
#pragma unroll
            for (int m = 0; m < MAPS; ++m) {
                __syncthreads();            // the rows of the map before this one have been taken in
                if (split > 0 && wave_on) {
                    float* mine = meet[wave - places][lane];
                    mine[0] = st.m[m];
                    mine[1] = st.l[m];
#pragma unroll
                    for (int t = 0; t < DVB; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) mine[2 + t * 4 + i] = st.o[m][t][i];
                }
                __syncthreads();
                if (split == 0 && wave_on)
                    for (int w = 1; w < splits; ++w) {          // in the waves' order
                        const float* its = meet[place + w * places - places][lane];
                        const float m_new = fmaxf(st.m[m], its[0]);
                        const float base = m_new == -INFINITY ? 0.f : m_new;
                        const float mine_by = expf(st.m[m] - base), its_by = expf(its[0] - base);
                        st.l[m] = fmaf(st.l[m], mine_by, its[1] * its_by);
#pragma unroll
                        for (int t = 0; t < DVB; ++t)
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                                st.o[m][t][i] = fmaf(st.o[m][t][i], mine_by, its[2 + t * 4 + i] * its_by);
                        st.m[m] = m_new;
                    }
            }
        }
        if (split == 0 && wave_on) {
            if (zsplits > 1) {
                const int passes = (group + 15) / 16;
                // [share][lane][map][numbers]: a lane's numbers in a row, which it reads back in wide loads
                float* mine = a.shares + ((((size_t)blockIdx.x * a.kv_heads + g) * passes + h0 / 16) * zsplits + z)
                                             * kWave * MAPS * share_floats<DVB>() + (size_t)lane * MAPS * share_floats<DVB>();
#pragma unroll
                for (int m = 0; m < MAPS; ++m) {
                    mine[m * share_floats<DVB>()] = st.m[m];
                    mine[m * share_floats<DVB>() + 1] = st.l[m];
#pragma unroll
                    for (int t = 0; t < DVB; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) mine[m * share_floats<DVB>() + 2 + t * 4 + i] = st.o[m][t][i];
                }
            } else {
                finish_column<DVB, MAPS>(st, a, tok, head, pos, lane);
            }
        }
    }
}

// Tiles of several tokens with their keys and values staged through LDS: all waves of the workgroup walk the same
// stage, which is fetched once for all of them, the next stage travelling through registers while this one is worked
// on.  A stage is `wave_blocks` blocks of 16 keys for every wave that shares a head's keys (one wave a head, or two
// where the group has four heads or fewer): two blocks a wave where a thread's share of a stage is two 16-byte pieces
// of keys and two of values at most, so that a stage's work outlasts the next one's trip from memory; else one.  Keys
// lie in LDS as rows with 16 bytes of padding, values transposed (a value entry's keys of the stage in a row, 16 bytes
// of padding): every operand is one read without bank conflicts.  Lone tokens are left to the kernel above.
constexpr int MB_STAGE_BLOCKS = 2;

template <int DSTEPS, int DVB, int MAPS>
__global__ __launch_bounds__(MB_THREADS) void masked_attention_bf16_staged_kernel(MaskedArgs a) {
    extern __shared__ __align__(16) unsigned char staged[];       // a stage; afterwards where split key ranges meet
    float (*meet)[kWave][DVB * 4 + 2] = reinterpret_cast<float (*)[kWave][DVB * 4 + 2]>(staged);
    const int* tile = a.tiles + 4 * blockIdx.x;
    const int t0 = tile[0], n = tile[1], r = tile[2], p0 = tile[3];
    if (n == 1) return;
    const int g = blockIdx.y, group = a.heads / a.kv_heads;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1), col = lane & 15, quad = lane >> 4;
    const int* table = a.block_table + (size_t)r * a.max_blocks;
    auto first_key = [&](int p) {
        int lo = 0;
        if (a.chunk > 0) lo = p - p % a.chunk;
        if (a.window > 0) lo = max(lo, p - a.window + 1);
        return lo;
    };
    int places = 1;
    while (places < group && places < MB_WAVES) places *= 2;
    const int splits = min(MB_WAVES / places, MB_STAGE_BLOCKS);      // waves that share a head's keys
    const int place = wave % places, split = wave / places;
    const int first = first_key(p0) / 16, last = (p0 + n - 1) / 16;
    const int stage_blocks = splits * a.wave_blocks;
    const int stages = (last - first + stage_blocks) / stage_blocks;
    const int seen_from = first_key(p0 + n - 1);        // every token of the tile sees the keys from here to p0
    const bool full_sizes = a.d == DSTEPS * 32 && a.dv == DVB * 16;
    const int d_all = MAPS * a.d;                               // a key row's entries of this kv head
    const int k_pitch = d_all * 2 + 16, v_pitch = stage_blocks * 32 + 16;           // bytes
    const int k_bytes = stage_blocks * 16 * k_pitch;
    const size_t k_row = (size_t)a.kv_heads * d_all;
    constexpr int PIECES = 2;                                   // a thread's pieces of each kind at most
    typedef int int4v __attribute__((ext_vector_type(4)));
    int4v kreg[PIECES], vreg[PIECES];
    // A thread's places in a stage are counted in units that the build knows (KP pieces a key row, DVB * 32 pieces a
    // block of values: no division by a size that only the launch knows); places beyond the real sizes stay empty.
    constexpr int KP = DSTEPS * 4 * MAPS, VP = DVB * 32, MAX_BLOCKS = 2 * MB_STAGE_BLOCKS;
    auto fetch = [&](int stage) {
        const int b0 = first + stage * stage_blocks;
        int page_of[MAX_BLOCKS], within_of[MAX_BLOCKS];         // the same for all threads
#pragma unroll
        for (int blk = 0; blk < MAX_BLOCKS; ++blk) {
            const int key0 = (b0 + blk) * 16;
            const bool there = blk < stage_blocks && b0 + blk <= last;
            page_of[blk] = there ? table[key0 / a.page_size] : -1;
            within_of[blk] = key0 % a.page_size;
        }
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int i = threadIdx.x + u * MB_THREADS;
            {
                const int key = i / KP, piece = i % KP, blk = key >> 4;
                int page = -1, within = 0;
#pragma unroll
                for (int x = 0; x < MAX_BLOCKS; ++x)
                    if (blk == x) { page = page_of[x]; within = within_of[x]; }
                if (page >= 0 && piece * 8 < d_all) {
                    const size_t row = (size_t)page * a.page_size + within + (key & 15);
                    kreg[u] = *reinterpret_cast<const int4v*>(a.k_cache + row * k_row + (size_t)g * d_all + piece * 8);
                }
            }
            {
                const int blk = i / VP, rem = i % VP, row = rem >> 1, half = rem & 1;
                int page = -1, within = 0;
#pragma unroll
                for (int x = 0; x < MAX_BLOCKS; ++x)
                    if (blk == x) { page = page_of[x]; within = within_of[x]; }
                if (page >= 0 && row < a.dv)
                    vreg[u] = *reinterpret_cast<const int4v*>(
                        a.v_cache + ((size_t)page * a.kv_heads * a.dv + (size_t)g * a.dv + row) * a.page_size + within + half * 8);
            }
        }
    };
    auto store = [&]() {
#pragma unroll
        for (int u = 0; u < PIECES; ++u) {
            const int i = threadIdx.x + u * MB_THREADS;
            {
                const int key = i / KP, piece = i % KP;
                if (key < stage_blocks * 16 && piece * 8 < d_all)
                    *reinterpret_cast<int4v*>(staged + key * k_pitch + piece * 16) = kreg[u];
            }
            {
                const int blk = i / VP, rem = i % VP, row = rem >> 1, half = rem & 1;
                if (blk < stage_blocks && row < a.dv)
                    *reinterpret_cast<int4v*>(staged + k_bytes + row * v_pitch + blk * 32 + half * 16) = vreg[u];
            }
        }
    };
    ColumnState<DVB, MAPS> st;
    for (int h0 = 0; h0 < group; h0 += places) {
        const int hh = h0 + place;
        const bool wave_on = hh < group && split < splits;
        const bool on = wave_on && col < n;
        const int head = g * group + (hh < group ? hh : 0);
        const int tok = t0 + (col < n ? col : 0);
        const int pos = on ? p0 + col : -1;
        const int lo = on ? first_key(pos) : 0;
        bf16x8 bq[MAPS][DSTEPS];
        load_queries<DSTEPS, MAPS>(bq, a, tok, head, pos, lane);
        const float bias1 = (a.r1 && pos >= 0) ? a.r1[head] : 0.f, bias2 = (a.r1 && pos >= 0) ? a.r2[head] : 0.f;
        clear_state<DVB, MAPS>(st);
        __syncthreads();                    // the pass before this one has read its last stage
        fetch(0);
        store();
        __syncthreads();
        for (int stage = 0; stage < stages; ++stage) {
            if (stage + 1 < stages) fetch(stage + 1);       // on its way while this stage is worked on
            for (int j = 0; j < a.wave_blocks; ++j) {
                const int blk = j * splits + split, b = first + stage * stage_blocks + blk;
                if (!wave_on || b > last) continue;
                bf16x8 ka[MAPS][DSTEPS];
                short4v va[DVB];
                const unsigned char* krow = staged + (blk * 16 + col) * k_pitch + quad * 16;
                const unsigned char* vrow = staged + k_bytes + col * v_pitch + blk * 32 + quad * 8;
                if (full_sizes) {           // the sizes the kernel is built for: no operand has empty places
#pragma unroll
                    for (int m = 0; m < MAPS; ++m)
#pragma unroll
                        for (int i = 0; i < DSTEPS; ++i)
                            ka[m][i] = *reinterpret_cast<const bf16x8*>(krow + (m * DSTEPS * 32 + i * 32) * 2);
#pragma unroll
                    for (int t = 0; t < DVB; ++t) va[t] = *reinterpret_cast<const short4v*>(vrow + t * 16 * v_pitch);
                } else {
#pragma unroll
                    for (int m = 0; m < MAPS; ++m)
#pragma unroll
                        for (int i = 0; i < DSTEPS; ++i) {
                            const int e = i * 32 + quad * 8;
#pragma unroll
                            for (int x = 0; x < 8; ++x) ka[m][i][x] = (__bf16)0.f;
                            if (e < a.d) ka[m][i] = *reinterpret_cast<const bf16x8*>(krow + (m * a.d + i * 32) * 2);
                        }
#pragma unroll
                    for (int t = 0; t < DVB; ++t) {
                        va[t] = short4v{0, 0, 0, 0};
                        if (t * 16 < a.dv) va[t] = *reinterpret_cast<const short4v*>(vrow + t * 16 * v_pitch);
                    }
                }
                block_step<DSTEPS, DVB, MAPS>(st, a, bq, ka, va, b * 16, pos, lo, bias1, bias2,
                                              b * 16 >= seen_from && b * 16 + 15 <= p0, lane);
            }
            __syncthreads();                    // every wave has read the stage
            if (stage + 1 < stages) store();
            __syncthreads();
        }
        if (splits > 1) {
#pragma unroll
            for (int m = 0; m < MAPS; ++m) {
                __syncthreads();
                if (split == 1 && wave_on) {
                    float* mine = meet[place][lane];
                    mine[0] = st.m[m];
                    mine[1] = st.l[m];
#pragma unroll
                    for (int t = 0; t < DVB; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) mine[2 + t * 4 + i] = st.o[m][t][i];
                }
                __syncthreads();
                if (split == 0 && wave_on) {
                    const float* its = meet[place][lane];
                    const float m_new = fmaxf(st.m[m], its[0]);
                    const float base = m_new == -INFINITY ? 0.f : m_new;
                    const float mine_by = expf(st.m[m] - base), its_by = expf(its[0] - base);
                    st.l[m] = fmaf(st.l[m], mine_by, its[1] * its_by);
#pragma unroll
                    for (int t = 0; t < DVB; ++t)
#pragma unroll
                        for (int i = 0; i < 4; ++i) st.o[m][t][i] = fmaf(st.o[m][t][i], mine_by, its[2 + t * 4 + i] * its_by);
                    st.m[m] = m_new;
                }
            }
        }
        if (split == 0 && wave_on) finish_column<DVB, MAPS>(st, a, tok, head, pos, lane);
    }
}

// One wave per lone token and kv head: the workgroups' shares taken in, in their order; then the columns' end.
template <int DVB, int MAPS>
__global__ __launch_bounds__(kWave) void masked_attention_bf16_join_kernel(MaskedArgs a) {
    const int* tile = a.tiles + 4 * blockIdx.x;
    const int t0 = tile[0], n = tile[1], p0 = tile[3];
    if (n != 1) return;
    const int g = blockIdx.y, group = a.heads / a.kv_heads, lane = threadIdx.x, col = lane & 15;
    const int passes = (group + 15) / 16;
    for (int h0 = 0; h0 < group; h0 += 16) {
        const bool on = h0 + col < group;
        const int head = g * group + (on ? h0 + col : 0);
        ColumnState<DVB, MAPS> st;
#pragma unroll
        for (int m = 0; m < MAPS; ++m) {
            st.m[m] = -INFINITY;
            st.l[m] = 0.f;
#pragma unroll
            for (int t = 0; t < DVB; ++t) st.o[m][t] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        for (int z = 0; z < a.zsplits; ++z) {
            const float* its = a.shares + ((((size_t)blockIdx.x * a.kv_heads + g) * passes + h0 / 16) * a.zsplits + z)
                                              * kWave * MAPS * share_floats<DVB>() + (size_t)lane * MAPS * share_floats<DVB>();
#pragma unroll
            for (int m = 0; m < MAPS; ++m) {
                const float* row = its + m * share_floats<DVB>();
                const float m_new = fmaxf(st.m[m], row[0]);
                const float base = m_new == -INFINITY ? 0.f : m_new;
                const float mine_by = expf(st.m[m] - base), its_by = expf(row[0] - base);
                st.l[m] = fmaf(st.l[m], mine_by, row[1] * its_by);
#pragma unroll
                for (int t = 0; t < DVB; ++t)
#pragma unroll
                    for (int i = 0; i < 4; ++i) st.o[m][t][i] = fmaf(st.o[m][t][i], mine_by, row[2 + t * 4 + i] * its_by);
                st.m[m] = m_new;
            }
        }
        finish_column<DVB, MAPS>(st, a, t0, head, on ? p0 : -1, lane);
    }
}

}  // namespace lc

using namespace lc;

static thread_local int g_staged = 1;

// Tests and tuning: whether tiles of several tokens may take the kernel that stages keys and values in LDS (for the
// calling thread).  Returns the setting before.
LC_API int lc_masked_attention_bf16_staged(int on) {
    const int before = g_staged;
    if (on >= 0) g_staged = on ? 1 : 0;
    return before;
}

// Whether the matrix-core kernel takes these sizes (else the general kernel serves them).
LC_API int lc_masked_attention_bf16_supported(int d, int dv, int page_size, int maps) {
    return d > 0 && d % 8 == 0 && d <= 128 && dv > 0 && dv % 16 == 0 && dv <= 128 && page_size > 0 && page_size % 16 == 0
           && (maps == 1 || maps == 2);
}

// float32 words of workspace for a step of `num_tiles` lone tokens whose keys are shared out over `zsplits` workgroups
LC_API long long lc_masked_attention_bf16_workspace(int num_tiles, int heads, int kv_heads, int maps, int dv, int zsplits) {
    if (num_tiles <= 0 || kv_heads <= 0 || heads % kv_heads || zsplits <= 1) return 0;
    const int dvb = dv <= 32 ? 2 : (dv <= 64 ? 4 : 8), passes = (heads / kv_heads + 15) / 16;
    return (long long)num_tiles * kv_heads * passes * zsplits * kWave * maps * (dvb * 4 + 2);
}

// tiles int32 [num_tiles, 4]: first token row, tokens (1..16), request, first position.  zsplits > 1 (a step of lone
// tokens only): every token's key blocks are shared out over that many workgroups, through `shares`
// (lc_masked_attention_bf16_workspace words)
LC_API int lc_masked_attention_bf16(const void* q, const void* k_cache, const void* v_cache, const int* tiles,
                                    int num_tiles, const int* block_table, int max_blocks, int page_size, int heads,
                                    int kv_heads, int maps, int d, int dv, float scale, int chunk, int window,
                                    const float* r1, const float* r2, const float* sink, float lambda, int unit_out,
                                    float eps, float out_scale, const float* gate, int gate_stride, int gate_column,
                                    void* out, float* shares, int zsplits, int any_portion, int any_lone,
                                    hipStream_t stream) {
    LC_CHECK(zsplits >= 1 && zsplits <= 64 && (zsplits == 1 || shares), "masked attention: bad shares");
    LC_CHECK(num_tiles >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && max_blocks > 0,
             "masked attention: bad sizes");
    LC_CHECK(lc_masked_attention_bf16_supported(d, dv, page_size, maps),
             "masked attention on the matrix cores: sizes d=%d dv=%d page=%d maps=%d are not taken", d, dv, page_size, maps);
    if (num_tiles == 0) return 0;
    LC_CHECK(q && k_cache && v_cache && tiles && block_table && out, "masked attention: null pointer");
    LC_CHECK((r1 == nullptr) == (r2 == nullptr), "masked attention: the bias needs both of its vectors");
    LC_CHECK(kv_heads <= 65535, "masked attention: too many kv heads");
    MaskedArgs a{(const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, tiles, block_table, max_blocks, page_size,
                 heads, kv_heads, d, dv, scale, chunk, window, r1, r2, sink, lambda, unit_out, eps, out_scale, gate,
                 gate_stride, gate_column, (bf16*)out, shares, zsplits, 0, 1};
    // tiles of several tokens go through the kernel that stages keys and values in LDS where a stage fits a thread's
    // two pieces of each kind
    const int group = heads / kv_heads;
    int places = 1;
    while (places < group && places < MB_WAVES) places *= 2;
    const int sharing = MB_WAVES / places < MB_STAGE_BLOCKS ? MB_WAVES / places : MB_STAGE_BLOCKS;
    const int dsteps_built = (d + 31) / 32 <= 2 ? 2 : 4, dvb_built = dv <= 32 ? 2 : (dv <= 64 ? 4 : 8);
    auto fits = [&](int blocks) {       // a thread's two places of each kind at most, in the units the kernels are built for
        return blocks * 16 * (dsteps_built * 4 * maps) <= 2 * MB_THREADS && blocks * dvb_built * 32 <= 2 * MB_THREADS;
    };
    const bool staged = any_portion && g_staged && fits(sharing);
    a.wave_blocks = fits(2 * sharing) ? 2 : 1;
    const int stage_blocks = sharing * a.wave_blocks;
    size_t staged_lds = (size_t)stage_blocks * 16 * (maps * d * 2 + 16) + (size_t)dv * (stage_blocks * 32 + 16);
    const size_t meet_lds = (size_t)(MB_WAVES / 2) * kWave * (8 * 4 + 2) * sizeof(float);    // the same memory, later
    if (staged_lds < meet_lds) staged_lds = meet_lds;
    a.lone_only = staged ? 1 : 0;
    const bool main_kernel = !staged || any_lone;
    const dim3 grid(num_tiles, kv_heads, zsplits), join_grid(num_tiles, kv_heads);
    const int dsteps = (d + 31) / 32, dvb = dv / 16;
#define LC_MB_AS(DS, VB, MP)                                                                                            \
    do {                                                                                                                \
        if (staged) masked_attention_bf16_staged_kernel<DS, VB, MP><<<join_grid, MB_THREADS, staged_lds, stream>>>(a);  \
        if (main_kernel) masked_attention_bf16_kernel<DS, VB, MP><<<grid, MB_THREADS, 0, stream>>>(a);                  \
        if (zsplits > 1) masked_attention_bf16_join_kernel<VB, MP><<<join_grid, kWave, 0, stream>>>(a);                 \
    } while (0)
#define LC_MB(DS, VB)                          \
    do {                                       \
        if (maps == 1) LC_MB_AS(DS, VB, 1);    \
        else LC_MB_AS(DS, VB, 2);              \
    } while (0)
#define LC_MB_DV(DS)                     \
    do {                                 \
        if (dvb <= 2) LC_MB(DS, 2);      \
        else if (dvb <= 4) LC_MB(DS, 4); \
        else LC_MB(DS, 8);               \
    } while (0)
    if (dsteps <= 2) LC_MB_DV(2);
    else LC_MB_DV(4);
#undef LC_MB_DV
#undef LC_MB
#undef LC_MB_AS
    LC_LAUNCH_CHECK("masked_attention_bf16");
    return 0;
}
