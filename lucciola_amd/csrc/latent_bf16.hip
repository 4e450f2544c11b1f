// Latent attention in bfloat16 on the matrix cores (v_mfma_f32_16x16x32_bf16), for latents of a
// multiple of 16 entries (up to 512) and rows [c | k_r] of a multiple of 8 (up to 576, of which up
// to 128 rotated).
//
// As in latent.hip every head of a token attends over the same cached rows, with the query in the
// latent's space; scores, maxima, exponentials and sums are float32, the weights are rounded to
// bfloat16 for the product with the rows (as the other matrix-core attention kernels do).
//
// A work item is a tile of the planner's list: up to 16 tokens in a row of one request (a piece
// of a prompt's portion), or one token (a decoding request).  A workgroup of four pairs of waves serves a
// tile and some heads: a pair has 16 query columns, which are the tile's tokens for one head (pair
// w: head h0 + w) or, for a lone token, 16 heads (pair w: heads h0 + 16 w ...).  All waves read
// the same keys: a stage of 32 cached rows is brought into LDS once, as rows (the operand of
// S^T = K . Q^T) and, its latent part, transposed ([entry][key], the operand of O^T = C^T . P^T),
// so that every operand is one 16-byte LDS read.  S^T leaves a lane with the keys 4 g + r of a
// query column, which is the layout that P^T needs as an operand: the weights never leave the
// registers.
//
// With few tiles the stages of a tile are shared out over gridDim.z workgroups that leave their
// maxima, sums and unnormalised rows in a workspace; a second kernel joins them in their order.
#include "common.h"

namespace lc {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int LM_THREADS = 512;       // eight waves: four pairs, a pair shares its query columns
constexpr int LM_STAGE = 32;          // keys of a stage
constexpr int LM_ROT_MOST = 128;      // rotated entries of a row, at most
constexpr int LM_KPAD = 8;            // bf16 of padding behind a staged row
constexpr int LM_VSTRIDE = LM_STAGE + 8;   // bf16 between two entries' key runs in the transposed stage

// (of a stage's 32 keys, lane group g's run of eight in the transposed stage is the keys 4 g ... 4 g + 3
// and 16 + 4 g ... 16 + 4 g + 3: the keys of its two score tiles, which its weights are made of)

// NR: tiles of 16 latent entries a wave keeps sums for; KS: steps of 32 row entries of a score
template <int NR, int KS>
__global__ __launch_bounds__(LM_THREADS) void latent_attention_bf16_kernel(
    const bf16* __restrict__ qa, int H, int R, int rot, const bf16* __restrict__ cache,
    const int* __restrict__ tiles, const int* __restrict__ block_table, int max_blocks, int page_size,
    float scale, int window, const float* __restrict__ sink, bf16* __restrict__ out, int splits,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int Dk = R + rot, Dp = KS * 32;
    const int kstride = Dp + LM_KPAD;                       // bf16 a staged row
    bf16* ks_lds = reinterpret_cast<bf16*>(lds_raw);        // [LM_STAGE][kstride]
    bf16* vt_lds = ks_lds + LM_STAGE * kstride;             // [R][LM_VSTRIDE]
    int* rows_lds = reinterpret_cast<int*>(vt_lds + (size_t)R * LM_VSTRIDE);    // [2][LM_STAGE]
    // a pair of waves has the same 16 query columns: both make the scores and weights (what one
    // would have to hand to the other costs more than making them twice), each sums one half of the
    // latent's entries, so that a wave's sums and queries fit half of a SIMD's registers and two
    // waves share every SIMD
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 7, half = (tid >> 6) & 1, col = lane & 15, g = lane >> 4;
    constexpr int NH = NR / 2;
    const int* tile = tiles + 4 * blockIdx.x;
    const int t0 = tile[0], ntok = tile[1], req = tile[2], p0 = tile[3];
    const bool lone = ntok == 1;
    const int h0 = blockIdx.y * (lone ? 64 : 4);
    if (h0 >= H) return;
    // this lane's query column
    const int q_tok = lone ? 0 : col, q_head = lone ? h0 + 16 * wave + col : h0 + wave;
    const bool q_live = q_tok < ntok && q_head < H;
    const bool wave_live = lone ? h0 + 16 * wave < H : h0 + wave < H;
    const int p_q = p0 + q_tok;
    // the keys the lane's column sees: q_lo .. q_hi (none for a column that is not there)
    const int q_hi = q_live ? p_q : -1;
    const int q_lo = window > 0 ? p_q - window + 1 : 0;
    const float scale_log2 = scale * 1.4426950408889634f;
    const int p_last = p0 + ntok - 1;
    const int j_lo = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    const int stages = (p_last - j_lo) / LM_STAGE + 1;
    const int per = (stages + splits - 1) / splits;
    const int s_begin = blockIdx.z * per, s_end = min(stages, s_begin + per);
    const int* table = block_table + (size_t)req * max_blocks;

    // the queries as operands: entries 32 ks + 8 g ... of the lane's column
    bf16x8 qf[KS];
    {
        const bf16* qrow = qa + ((size_t)(t0 + (q_live ? q_tok : 0)) * H + (q_live ? q_head : 0)) * Dk;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int e = s * 32 + 8 * g;
            if (q_live && wave_live && e < Dk) qf[s] = *reinterpret_cast<const bf16x8*>(qrow + e);
            else
#pragma unroll
                for (int i = 0; i < 8; ++i) qf[s][i] = static_cast<bf16>(0.f);
        }
    }
    // the padding behind the rows' entries counts as zero in every score
    for (int i = tid; i < LM_STAGE * (Dp - Dk); i += LM_THREADS) {
        const int key = i / (Dp - Dk), e = Dk + i % (Dp - Dk);
        ks_lds[key * kstride + e] = static_cast<bf16>(0.f);
    }
    floatx4 o[NH];                                          // entries 16 (half NH + d) ... of the latent
#pragma unroll
    for (int d = 0; d < NH; ++d) o[d] = floatx4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // where the keys of a stage lie (page * page size + offset): a key
    // behind the tile's last is that last key once more (finite, and no query sees it)
    auto row_of = [&](int j) {
        j = min(j, p_last);
        return table[j / page_size] * page_size + j % page_size;
    };
    // Staging.  A thread brings, of the latent part, eight entries of four keys: one half of a lane
    // group's run of eight (R / 8 x 8 such pieces of work, at most one a thread), and stores them
    // twice: as they are into the rows, and transposed (for each entry its half of the run as one
    // 8-byte piece).  Of the rotated part behind the latent it brings single 16-byte pieces.  All of
    // it is asked for a stage ahead and travels while the stage before is multiplied.
    const int gg = tid & 3, hh = (tid >> 2) & 1, dp = tid >> 3;
    const bool has_c = dp * 8 < R;
    const int rot_pieces = rot / 8;                         // 16-byte pieces of a row's rotated part
    constexpr int RP = LM_STAGE * (LM_ROT_MOST / 8) / LM_THREADS;             // such pieces a thread, at most
    bf16x8 in[4], extra[RP];
    int ex_key[RP], ex_piece[RP];
#pragma unroll
    for (int u = 0; u < RP; ++u) {
        const int i = tid + u * LM_THREADS;
        ex_key[u] = rot_pieces ? i / rot_pieces : LM_STAGE;
        ex_piece[u] = rot_pieces ? i - ex_key[u] * rot_pieces : 0;
    }
    auto ask = [&](const int* rows) {
        if (has_c)
#pragma unroll
            for (int k = 0; k < 4; ++k)
                in[k] = *reinterpret_cast<const bf16x8*>(cache + (size_t)rows[16 * hh + 4 * gg + k] * Dk + dp * 8);
#pragma unroll
        for (int u = 0; u < RP; ++u)
            if (ex_key[u] < LM_STAGE)
                extra[u] = *reinterpret_cast<const bf16x8*>(cache + (size_t)rows[ex_key[u]] * Dk + R + ex_piece[u] * 8);
    };
    // the rows of stage s + 2 are looked up while stage s is staged, wait in a register and reach
    // LDS at the top of stage s + 1, whose loads for stage s + 2 read them: no look-up is waited for
    int row_ahead = 0;
    if (s_begin < s_end) {
        if (tid < LM_STAGE) {
            rows_lds[tid] = row_of(j_lo + s_begin * LM_STAGE + tid);
            if (s_begin + 1 < s_end) row_ahead = row_of(j_lo + (s_begin + 1) * LM_STAGE + tid);
        }
        __syncthreads();
        ask(rows_lds);
    }
    for (int s = s_begin; s < s_end; ++s) {
        const int c0 = j_lo + s * LM_STAGE;
        int* rows_next = rows_lds + ((s + 1 - s_begin) & 1) * LM_STAGE;
        __syncthreads();                                    // the stage before has been read
        if (tid < LM_STAGE && s + 1 < s_end) {
            rows_next[tid] = row_ahead;
            if (s + 2 < s_end) row_ahead = row_of(c0 + 2 * LM_STAGE + tid);
        }
        if (has_c) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
                *reinterpret_cast<bf16x8*>(ks_lds + (16 * hh + 4 * gg + k) * kstride + dp * 8) = in[k];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                bf16x4 run;
#pragma unroll
                for (int k = 0; k < 4; ++k) run[k] = in[k][e];
                *reinterpret_cast<bf16x4*>(vt_lds + (dp * 8 + e) * LM_VSTRIDE + gg * 8 + hh * 4) = run;
            }
        }
#pragma unroll
        for (int u = 0; u < RP; ++u)
            if (ex_key[u] < LM_STAGE)
                *reinterpret_cast<bf16x8*>(ks_lds + ex_key[u] * kstride + R + ex_piece[u] * 8) = extra[u];
        __syncthreads();
        if (s + 1 < s_end) ask(rows_next);                  // the next stage's rows travel while this one is multiplied
        if (!wave_live) continue;
        // S^T = K . Q^T: two tiles of 16 keys.  The operands of a batch of products are all asked of
        // LDS before the first product (a wave that is alone on its SIMD would otherwise wait for
        // every read in turn), and the two tiles' products alternate
        floatx4 sc[2];
        sc[0] = sc[1] = floatx4{0.f, 0.f, 0.f, 0.f};
        {
            const bf16* krow = ks_lds + col * kstride + 8 * g;
            constexpr int QB = 3;                           // steps of 32 entries a batch, for both tiles
#pragma unroll
            for (int x0 = 0; x0 < KS; x0 += QB) {
                bf16x8 ka[2][QB];
#pragma unroll
                for (int i = 0; i < QB; ++i)
                    if (x0 + i < KS)
#pragma unroll
                        for (int kt = 0; kt < 2; ++kt)
                            ka[kt][i] = *reinterpret_cast<const bf16x8*>(krow + kt * 16 * kstride + (x0 + i) * 32);
#pragma unroll
                for (int i = 0; i < QB; ++i)
                    if (x0 + i < KS)
#pragma unroll
                        for (int kt = 0; kt < 2; ++kt)
                            sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kt][i], qf[x0 + i], sc[kt], 0, 0, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * QB, 0);      // the batch's LDS reads, then its products
                __builtin_amdgcn_sched_group_barrier(0x008, 2 * QB, 0);
            }
        }
        // the lane holds the keys c0 + 16 kt + 4 g + r of its column; scores in units of log 2, so that
        // every exponential is one instruction
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = c0 + 16 * kt + 4 * g + r;
                sc[kt][r] = (j >= q_lo && j <= q_hi) ? sc[kt][r] * scale_log2 : -INFINITY;
                mx = fmaxf(mx, sc[kt][r]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
        mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
        const float m_new = fmaxf(m_run, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);   // 0 while the column has seen no key (its sums are 0)
        float sum = 0.f;
        bf16x8 pb;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float pj = __builtin_amdgcn_exp2f(sc[kt][r] - m_safe);
                sum += pj;
                pb[4 * kt + r] = static_cast<bf16>(pj);
            }
        sum += __shfl_xor(sum, 16, kWave);
        sum += __shfl_xor(sum, 32, kWave);
        l_run = fmaf(l_run, alpha, sum);
        m_run = m_new;
        const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
        // O^T += C^T . P^T, the operands again a batch at a time
        if (rescale)
#pragma unroll
            for (int d = 0; d < NH; ++d)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[d][r] *= alpha;
        {
            constexpr int PB = NH < 8 ? NH : 8;
            const bf16* vrow = vt_lds + ((half * NH) * 16 + col) * LM_VSTRIDE + 8 * g;
#pragma unroll
            for (int d0 = 0; d0 < NH; d0 += PB) {
                bf16x8 va[PB];
#pragma unroll
                for (int i = 0; i < PB; ++i)
                    if ((half * NH + d0 + i) * 16 < R) va[i] = *reinterpret_cast<const bf16x8*>(vrow + (d0 + i) * 16 * LM_VSTRIDE);
#pragma unroll
                for (int i = 0; i < PB; ++i)
                    if ((half * NH + d0 + i) * 16 < R)
                        o[d0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[i], pb, o[d0 + i], 0, 0, 0);
            }
        }
    }
    if (!wave_live || !q_live) return;
    // the lane holds the entries 16 d + 4 g + r of its column
    const size_t qi = (size_t)(t0 + q_tok) * H + q_head;
    if (splits == 1) {
        float inv = 1.f / l_run;
        if (sink) {
            // one more term in the denominator: exp(sink), a key with that score and no value (the
            // maxima are in units of log 2)
            const float s2 = sink[q_head] * 1.4426950408889634f;
            const float m_all = fmaxf(m_run, s2);
            const float keep = __builtin_amdgcn_exp2f(m_run - m_all);
            inv = keep / fmaf(l_run, keep, __builtin_amdgcn_exp2f(s2 - m_all));
        }
#pragma unroll
        for (int d = 0; d < NH; ++d)
            if ((half * NH + d) * 16 < R) {
                bf16* dst = out + qi * R + (half * NH + d) * 16 + 4 * g;
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[r] = static_cast<bf16>(o[d][r] * inv);
            }
    } else {
        float* dst = part_o + (qi * splits + blockIdx.z) * R;
#pragma unroll
        for (int d = 0; d < NH; ++d)
            if ((half * NH + d) * 16 < R)
#pragma unroll
                for (int r = 0; r < 4; ++r) dst[(half * NH + d) * 16 + 4 * g + r] = o[d][r];
        if (g == 0 && half == 0) {
            part_ml[(qi * splits + blockIdx.z) * 2] = m_run;
            part_ml[(qi * splits + blockIdx.z) * 2 + 1] = l_run;
        }
    }
}

// One workgroup per (token, head): the shares' sums, taken in from the first.
__global__ void latent_attention_join_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                             int splits, int R, int H, const float* __restrict__ sink,
                                             bf16* __restrict__ out) {
    __shared__ float weight[64];
    __shared__ float total;
    const size_t qi = blockIdx.x;
    if (threadIdx.x < 64) {
        const int z = threadIdx.x;
        const float m = z < splits ? part_ml[(qi * splits + z) * 2] : -INFINITY;
        // the head's sink counts as one more share: maximum sink, sum 1, no row
        const float s2 = sink ? sink[qi % H] * 1.4426950408889634f : -INFINITY;
        const float M = fmaxf(wave_max(m), s2);
        const float w = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - M);     // the maxima are in units of log 2
        weight[z] = w;
        const float L = wave_sum(z < splits ? part_ml[(qi * splits + z) * 2 + 1] * w : 0.f);
        if (z == 0) total = L + (sink ? __builtin_amdgcn_exp2f(s2 - M) : 0.f);
    }
    __syncthreads();
    const float inv = 1.f / total;
    for (int d = threadIdx.x; d < R; d += blockDim.x) {
        float acc = 0.f;
        for (int z = 0; z < splits; ++z) acc = fmaf(part_o[(qi * splits + z) * R + d], weight[z], acc);
        out[qi * R + d] = static_cast<bf16>(acc * inv);
    }
}

static bool shape_of(int R, int rot, int* nr, int* ks) {
    const int Dk = R + rot;
    if (R <= 0 || R % 16 || Dk % 8 || R > 512 || Dk > 576 || rot > LM_ROT_MOST) return false;
    const int need_nr = R / 16, need_ks = (Dk + 31) / 32;
    const int classes[4][2] = {{4, 4}, {8, 8}, {16, 12}, {32, 18}};
    for (auto& c : classes)
        if (need_nr <= c[0] && need_ks <= c[1]) { *nr = c[0]; *ks = c[1]; return true; }
    return false;
}

}  // namespace lc

using namespace lc;

// Whether the matrix-core kernel serves these sizes.
LC_API int lc_latent_bf16_supported(int R, int rot) {
    int nr, ks;
    return shape_of(R, rot, &nr, &ks) ? 1 : 0;
}

// Shares the stages of a tile are cut into: from the number of workgroups without shares and
// the most keys a tile can see.
LC_API int lc_latent_bf16_splits(int workgroups, int max_keys) {
    if (workgroups <= 0) return 1;
    const int stages = (max_keys + LM_STAGE - 1) / LM_STAGE;
    int want = (device_cus() + workgroups - 1) / workgroups;          // one workgroup a CU: a CU holds no more
    if (want > stages / 2) want = stages / 2;                          // two stages a share at least
    if (want > 64) want = 64;
    return want < 2 ? 1 : want;
}

// qa [T, H, R + rot], cache [slots, R + rot] -> out [T, H, R].  tiles [NT, 4]: first token row, tokens
// (1 to 16), request, first position.  any_portion: whether a tile has more than one token (the
// grid then has a workgroup per four heads).  splits > 1: part_o [T H splits R] and part_ml [T H
// splits 2] float32.
LC_API int lc_latent_attention_bf16(const void* qa, int T, int H, int R, int rot, const void* cache, const int* tiles,
                                    int num_tiles, int any_portion, const int* block_table, int max_blocks,
                                    int page_size, float scale, int window, const float* sink, void* out, int splits,
                                    float* part_o, float* part_ml, hipStream_t stream) {
    int nr = 0, ks = 0;
    LC_CHECK(shape_of(R, rot, &nr, &ks), "latent attention: the matrix-core kernel does not take a latent of %d + %d", R, rot);
    LC_CHECK(T >= 0 && H > 0 && num_tiles >= 0 && page_size > 0 && max_blocks > 0 && splits >= 1 && splits <= 65535,
             "latent attention: bad sizes");
    if (T == 0 || num_tiles == 0) return 0;
    LC_CHECK(qa && cache && tiles && block_table && out, "latent attention: null pointer");
    LC_CHECK(splits == 1 || (part_o && part_ml), "latent attention: shares need a workspace");
    const int blocks_y = any_portion ? (H + 3) / 4 : (H + 63) / 64;
    LC_CHECK(blocks_y <= 65535, "latent attention: too many heads (%d)", H);
    const dim3 grid(num_tiles, blocks_y, splits);
    const size_t lds = sizeof(bf16) * ((size_t)LM_STAGE * (ks * 32 + LM_KPAD) + (size_t)R * LM_VSTRIDE) +
                       sizeof(int) * 2 * LM_STAGE;
#define LC_LM_LAUNCH(NR, KS)                                                                                       \
    do {                                                                                                           \
        if (lds > 64 * 1024)                                                                                       \
            LC_CHECK(hipFuncSetAttribute((const void*)latent_attention_bf16_kernel<NR, KS>,                        \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,      \
                     "latent attention: %zu bytes of LDS refused", lds);                                           \
        latent_attention_bf16_kernel<NR, KS><<<grid, LM_THREADS, lds, stream>>>(                                    \
            (const bf16*)qa, H, R, rot, (const bf16*)cache, tiles, block_table, max_blocks, page_size, scale, window, \
            sink, (bf16*)out, splits, part_o, part_ml);                                                               \
    } while (0)
    if (nr == 4) LC_LM_LAUNCH(4, 4);
    else if (nr == 8) LC_LM_LAUNCH(8, 8);
    else if (nr == 16) LC_LM_LAUNCH(16, 12);
    else LC_LM_LAUNCH(32, 18);
#undef LC_LM_LAUNCH
    LC_LAUNCH_CHECK("latent_attention_bf16");
    if (splits > 1) {
        latent_attention_join_kernel<<<T * H, 256, 0, stream>>>(part_o, part_ml, splits, R, H, sink, (bf16*)out);
        LC_LAUNCH_CHECK("latent_attention_join");
    }
    return 0;
}
