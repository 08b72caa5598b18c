// bf16 paged attention on the matrix cores for mixers whose scores carry a distance bias, whose
// softmax may have a term without a value (a sink), and whose values may have another size than
// their keys. One kernel serves prompts, portions, mixed steps and decode steps.
//
// Cache layout as everywhere in this folder: keys [pages, Hkv, 16, hd], values [pages, Hkv, hdv, 16]
// (transposed inside the page), page size 16. Token t of the packed batch reads the keys
// [kv_lo[t], kv_hi[t]) of its row; the step's own keys are already in the cache, and queries and
// keys come normalised where the mixer normalises them.
//
// The score of query t (place p = positions[t]) of head h against the key at place j is
//     scale * (q . k) - slopes[h] * (p - j) + table[h, min(p - j, bias_len - 1)]     (slopes and table optional)
// (the table: a learned bias per head and distance that is constant from some distance on, fp32 [H, bias_len]);
// and the weights are exp(s_j) / (sum_j exp(s_j) [+ exp(sink)]): fp32 throughout; the weights enter
// the value product as bf16, sums in fp32.
//
// Further forms of the same loop, for mixers that are attention with a twist:
//  * sinks (fp32 [H]): the valueless term's score per head instead of one number;
//  * keep_first: a query also sees the keys [0, min(keep_first, kv_lo)) of its row, before its window
//    (their tiles are taken ahead of the window's);
//  * maps > 1: query and key heads come in groups of `maps` neighbours, map m of a query head reads map m of
//    its key head, and all maps of a key head share one value head (H and Hkv count maps, the value cache has
//    Hkv / maps heads);
//  * values_in_keys: a key's value is the first hdv channels of its key row (a cache of latents that are keys
//    and values at once); the value operand is then gathered from the key page;
//  * out_f32: outputs leave as fp32;
//  * softcap > 0: scale * (q . k) passes through softcap * tanh(. / softcap) before the other terms are added;
//  * gate_per_head: the output gate holds one number per head ([n, H]) instead of one per channel.
//
// A decode step of few rows has few workgroups. With n_splits > 1 a row's tiles of keys are dealt out over that many
// workgroups in contiguous runs; each leaves its unnormalised outputs, reference point and sum in `partial`
// (fp32 [tokens, H, n_splits, hdv + 2]), and attn_biased_finish_kernel merges them (the sink, the gate and the
// output's type are then its business).
//
// Heads wider than 128 channels (latent rows of several hundred numbers) take the same loop in its wide form (NK = 0):
// the head size is a run-time number, the queries of the workgroup's 32 columns lie in LDS instead of registers (every
// wave reads them from there, 16 bytes a lane and step), keys are streamed step by step, and a workgroup owns a slice of
// 128 value channels (blockIdx.z counts the slices; every slice computes the scores again, which costs little where
// the keys are what is waited for).
//
// A workgroup owns 32 columns of the score product and one kv head. In a step with prompt portions a
// column is a query of a block of 32 consecutive tokens of one row and one query head (the host lists the
// blocks); in a decode step, where every row has one token, the columns are the query heads that share the
// kv head (up to 32), so that the row's keys and values are read once for all of them. Its waves take the
// tiles of 32 keys (two pages) in turn. Scores are computed transposed, S^T = K Q^T, with
// v_mfma_f32_32x32x16_bf16: a lane then holds 16 scores of ONE column, so the softmax is in-lane work
// plus one exchange with the lane 32 away. The key rows are fed to the product with bits 2 and 3 of the row index
// swapped: the 8 weights a lane holds per page are then those of 8 consecutive keys, which is, as they stand,
// the column operand of O^T += V^T P^T, whose row operand is one 16-byte load from the transposed value
// page. The outputs are rescaled only when some column's maximum has grown by more than 2^8. Waves merge
// through LDS in a tree.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 ab_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 ab_bf16x4;
typedef __attribute__((ext_vector_type(16))) float ab_floatx16;

constexpr int AB_PAGE = 16;
constexpr int AB_TILE = 32;                 // keys per tile: two pages
constexpr int AB_COLS = 32;                 // columns (queries) per workgroup
constexpr float AB_SLACK = 8.0f;            // powers of two a maximum may grow before the outputs are rescaled
constexpr float AB_LOG2E = 1.4426950408889634f;

__device__ __forceinline__ float ab_max_halves(float x) {
    typedef __attribute__((ext_vector_type(2))) unsigned ab_u2;
    const ab_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float ab_sum_halves(float x) {
    typedef __attribute__((ext_vector_type(2))) unsigned ab_u2;
    const ab_u2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// NK: 16-channel steps of a query/key head (hd = 16 NK; NK = 0: hd_wide channels, see above); NV: 32-channel blocks of a
// value head (hdv <= 32 NV, or, in the wide form, the slice of the value head that blockIdx.z names).
// heads_per_block: 1 = the columns are consecutive tokens of a block of queries (qblk_row / qblk_tok list the blocks,
// grid (H, blocks)); > 1 = a decode step, the columns are that many query heads of one kv head of token blockIdx.y
// (grid (Hkv * ceil(G / heads_per_block), tokens)).
template <int NK, int NV>
__global__ void __launch_bounds__(512)
attn_biased_kernel(const bf16_t* __restrict__ q, long q_row_stride, const bf16_t* __restrict__ k_cache,
                   const bf16_t* __restrict__ v_cache, const int* __restrict__ block_table, int max_pages,
                   const int* __restrict__ qblk_row, const int* __restrict__ qblk_tok, const int* __restrict__ cu_q,
                   const int* __restrict__ token_row, const int* __restrict__ kv_lo, const int* __restrict__ kv_hi,
                   const int* __restrict__ positions, const float* __restrict__ slopes, bf16_t* __restrict__ out,
                   long out_row_stride, float scale, int H, int Hkv, int hdv, int heads_per_block, int has_sink,
                   float sink_score, const float* __restrict__ bias_table, int bias_len, const bf16_t* __restrict__ gate,
                   long gate_row_stride, const float* __restrict__ sinks, int keep_first, int maps, int values_in_keys,
                   int out_f32, int hd_wide, int n_splits, float* __restrict__ partial, float softcap, int gate_per_head) {
    constexpr bool WIDE = NK == 0;
    const int HD = WIDE ? hd_wide : NK * 16;
    const int v0 = WIDE ? blockIdx.z * (NV * 32) : 0;     // the first value channel of this workgroup's slice
    constexpr int REC = 16 * NV + 2;            // floats a lane hands over at a merge: its outputs, m and l
    extern __shared__ float mrg[];              // [waves / 2][REC][64]
    const int n_waves = blockDim.x / KA_WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / KA_WAVE), lane = threadIdx.x % KA_WAVE;
    const int col = lane % 32, half = lane / 32;
    const int G = H / Hkv;
    int kvh, head, tok, row;
    bool live;
    int split = 0;
    if (heads_per_block > 1) {
        const int groups = (G + heads_per_block - 1) / heads_per_block;
        const int bx = blockIdx.x % (Hkv * groups);
        split = blockIdx.x / (Hkv * groups);
        kvh = bx / groups;
        const int hq = (bx % groups) * heads_per_block + col;
        live = col < heads_per_block && hq < G;
        // (maps == 1: head kvh * G + hq)
        head = ((kvh / maps) * G + (live ? hq : 0)) * maps + kvh % maps;
        tok = blockIdx.y;
        row = token_row[tok];
    } else {
        head = blockIdx.x;
        kvh = (head / maps / G) * maps + head % maps;
        const int blk = blockIdx.y;
        row = qblk_row[blk];
        const int tok_end = cu_q[row + 1];
        if (qblk_tok[blk] >= tok_end) return;          // (the unused end of a list of fixed length)
        tok = qblk_tok[blk] + col;
        live = tok < tok_end;
        if (!live) tok = tok_end - 1;
    }
    const int hi = live ? kv_hi[tok] : 0;
    const int lo = live ? (kv_lo ? kv_lo[tok] : 0) : 0;
    // the block's range of keys, and the part of it that every live column sees whole
    int blk_hi = ka_lanes_reduce<1, KA_WAVE>(hi, KaIntMax{});
    int blk_lo = ka_lanes_reduce<1, KA_WAVE>(live && hi > lo ? lo : 0x7fffffff, KaIntMin{});
    int min_hi = ka_lanes_reduce<1, KA_WAVE>(live ? hi : 0x7fffffff, KaIntMin{});
    int max_lo = ka_lanes_reduce<1, KA_WAVE>(live ? lo : 0, KaIntMax{});
    blk_hi = __builtin_amdgcn_readfirstlane(blk_hi);
    blk_lo = __builtin_amdgcn_readfirstlane(blk_lo);
    min_hi = __builtin_amdgcn_readfirstlane(min_hi);
    max_lo = __builtin_amdgcn_readfirstlane(max_lo);

    // queries: the column operand of the score product, held for the whole loop
    ab_bf16x8 qreg[WIDE ? 1 : NK];
    ab_bf16x8* q_lds = reinterpret_cast<ab_bf16x8*>(mrg + (size_t)(n_waves / 2) * REC * KA_WAVE);     // [hd / 16][64]
    {
        const bf16_t* qp = q + (size_t)tok * q_row_stride + (size_t)head * HD + half * 8;
        if constexpr (WIDE) {
            for (int c = wave; c < HD / 16; c += n_waves) q_lds[c * KA_WAVE + lane] = *reinterpret_cast<const ab_bf16x8*>(qp + c * 16);
            __syncthreads();
        } else {
#pragma unroll
            for (int c = 0; c < NK; ++c) qreg[c] = *reinterpret_cast<const ab_bf16x8*>(qp + c * 16);
        }
    }
    const float slope2 = slopes ? slopes[head] * AB_LOG2E : 0.f;     // in powers of two, like everything below
    // (a cap: the product is first brought to score / cap, whose tanh times cap, in powers of two, is the score)
    const float scale2 = softcap > 0.f ? scale / softcap * (2.0f * AB_LOG2E) : scale * AB_LOG2E;
    const float cap2 = softcap * AB_LOG2E;
    const int place = (slopes || bias_table) ? positions[tok] : 0;
    const float* bias_row = bias_table ? bias_table + (size_t)head * bias_len : nullptr;
    const float bias_far2 = bias_row ? bias_row[bias_len - 1] * AB_LOG2E : 0.f;
    const float sink2 = (sinks ? sinks[head] : sink_score) * AB_LOG2E;
    const int vh = kvh / maps, Hv = Hkv / maps;

    float m = has_sink ? sink2 : -INFINITY;     // reference point of this lane's column (the same in both halves)
    float l = 0.f;                              // this lane's share of the column's sum
    ab_floatx16 o[NV];
#pragma unroll
    for (int b = 0; b < NV; ++b)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[b][i] = 0.f;

    const int* table = block_table + (size_t)row * max_pages;
    // the key this lane loads for the score product: row `col` of the product is key perm(col) of the tile
    const int krow = (col & 0x13) | ((col & 4) << 1) | ((col & 8) >> 1);
    const int kpage_in_tile = krow >> 4, kslot = krow & 15;
    const size_t k_head = (size_t)kvh * AB_PAGE * HD, k_page = (size_t)Hkv * AB_PAGE * HD;
    const size_t v_page = (size_t)Hv * hdv * AB_PAGE;
    // the value rows (channels) this lane loads: clamped into the head where the last block is not full
    int vch[NV];
#pragma unroll
    for (int b = 0; b < NV; ++b) vch[b] = min(v0 + b * 32 + col, hdv - 1);

    if (blk_lo < blk_hi) {
        const int first_tile = blk_lo / AB_TILE, last_tile = (blk_hi - 1) / AB_TILE;
        // tiles of kept first keys that lie wholly before the window's first tile come ahead of the window's
        const int kept_tiles = min((min(keep_first, blk_lo) + AB_TILE - 1) / AB_TILE, first_tile);
        const int n_tiles = kept_tiles + last_tile - first_tile + 1;
        const int per_split = (n_tiles + n_splits - 1) / n_splits;
        const int turn_end = min(n_tiles, (split + 1) * per_split);
        for (int turn = split * per_split + wave; turn < turn_end; turn += n_waves) {
            const int tile = turn < kept_tiles ? turn : first_tile + (turn - kept_tiles);
            const int base = tile * AB_TILE;
            // pages of the tile (a page the row has given back, or none: any page, its keys are masked)
            int pg[2];
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                const int e = table[min(tile * 2 + p, max_pages - 1)];
                pg[p] = e < 0 ? 0 : e;
            }
            ab_bf16x8 kr[WIDE ? 1 : NK];
            const bf16_t* kp = k_cache + (size_t)pg[kpage_in_tile] * k_page + k_head + (size_t)kslot * HD + half * 8;
            if constexpr (!WIDE) {
#pragma unroll
                for (int c = 0; c < NK; ++c) kr[c] = *reinterpret_cast<const ab_bf16x8*>(kp + c * 16);
            }
            ab_bf16x8 vr[2][NV];
            if (values_in_keys) {
                // eight consecutive keys of one channel: a column of the row-major key page
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    const bf16_t* vp = k_cache + (size_t)pg[p] * k_page + k_head + (size_t)(half * 8) * HD;
#pragma unroll
                    for (int b = 0; b < NV; ++b)
#pragma unroll
                        for (int e = 0; e < 8; ++e) vr[p][b][e] = vp[(size_t)e * HD + vch[b]];
                }
            } else {
#pragma unroll
                for (int p = 0; p < 2; ++p)
#pragma unroll
                    for (int b = 0; b < NV; ++b)
                        vr[p][b] = *reinterpret_cast<const ab_bf16x8*>(v_cache + (size_t)pg[p] * v_page +
                                                                       ((size_t)vh * hdv + vch[b]) * AB_PAGE + half * 8);
            }
            ab_floatx16 s;
#pragma unroll
            for (int i = 0; i < 16; ++i) s[i] = 0.f;
            if constexpr (WIDE) {

                for (int c = 0; c < HD / 16; ++c)
                    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const ab_bf16x8*>(kp + c * 16),
                                                                q_lds[c * KA_WAVE + lane], s, 0, 0, 0);
            } else {
#pragma unroll
                for (int c = 0; c < NK; ++c) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kr[c], qreg[c], s, 0, 0, 0);
            }
            // register i of this lane: key base + (i / 8) * 16 + half * 8 + i % 8 of the lane's column
            const int j0 = base + half * 8;
            const float bias0 = -slope2 * (float)(place - j0);          // (an integer distance: exact)
            const bool whole = turn >= kept_tiles && base >= max_lo && base + AB_TILE <= min_hi;
            if (!whole) {
                // Keys that no column of the block sees (slots behind the row's last key, pages given back) may hold
                // anything, a NaN included, and a weight of 0 does not clear that in a product: their values are zeroed.
#pragma unroll
                for (int p = 0; p < 2; ++p)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int j = base + p * AB_PAGE + half * 8 + e;
                        if ((j < blk_lo && j >= keep_first) || j >= blk_hi) {
#pragma unroll
                            for (int b = 0; b < NV; ++b) vr[p][b][e] = (bf16_t)0.f;
                        }
                    }
            }
            // a tile that lies, for every column, at least as far back as the table's last entry: one bias for all its keys
            const bool near_tile = bias_row != nullptr &&
                __builtin_amdgcn_ballot_w64(place - (base + AB_TILE - 1) < bias_len - 1) != 0;
            float tile_max = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int off = (i / 8) * 16 + i % 8;
                float x;
                if (softcap > 0.f) {
                    // tanh(z) = 1 - 2 / (e^(2z) + 1), with s * scale2 = 2 z log2(e)
                    const float e = __builtin_amdgcn_exp2f(s[i] * scale2);
                    x = fmaf(cap2, 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f), fmaf(slope2, (float)off, bias0));
                } else {
                    x = fmaf(s[i], scale2, fmaf(slope2, (float)off, bias0));
                }
                if (near_tile) x = fmaf(bias_row[min(max(place - (j0 + off), 0), bias_len - 1)], AB_LOG2E, x);
                else x += bias_far2;
                if (!whole) {
                    const int j = j0 + off;
                    if ((j < lo && j >= keep_first) || j >= hi) x = -INFINITY;
                }
                s[i] = x;
                tile_max = fmaxf(tile_max, x);
            }
            tile_max = ab_max_halves(tile_max);
            // the reference point moves only when some column's maximum has outgrown it by 2^slack
            if (__builtin_amdgcn_ballot_w64(tile_max > m + AB_SLACK) != 0) {
                const float m_new = fmaxf(m, tile_max);
                const float corr = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
                l *= corr;
#pragma unroll
                for (int b = 0; b < NV; ++b)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o[b][i] *= corr;
                m = m_new;
            }
            const float ref = m == -INFINITY ? 0.f : m;
            ab_bf16x8 pb[2];
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float p = __builtin_amdgcn_exp2f(s[i] - ref);      // (a masked key: exp2(-inf) = 0)
                sum += p;
                pb[i / 8][i % 8] = (bf16_t)p;
            }
            l += sum;
#pragma unroll
            for (int p = 0; p < 2; ++p)
#pragma unroll
                for (int b = 0; b < NV; ++b) o[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vr[p][b], pb[p], o[b], 0, 0, 0);
        }
    }
    l = ab_sum_halves(l);                       // the column's whole sum, in both of its lanes

    // merge the waves in a tree: at step s the waves with bit s set hand over to the wave 2^s below
    for (int step = 1; step < n_waves; step <<= 1) {
        const bool gives = (wave & (2 * step - 1)) == step, takes = (wave & (2 * step - 1)) == 0 && wave + step < n_waves;
        float* slot = mrg + (size_t)(wave / (2 * step)) * REC * KA_WAVE;
        if (gives) {
#pragma unroll
            for (int b = 0; b < NV; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) slot[(b * 16 + i) * KA_WAVE + lane] = o[b][i];
            slot[(16 * NV) * KA_WAVE + lane] = m;
            slot[(16 * NV + 1) * KA_WAVE + lane] = l;
        }
        __syncthreads();
        if (takes) {
            const float m2 = slot[(16 * NV) * KA_WAVE + lane], l2 = slot[(16 * NV + 1) * KA_WAVE + lane];
            const float m_new = fmaxf(m, m2);
            const float c1 = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - m_new);
            const float c2 = m_new == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m2 - m_new);
#pragma unroll
            for (int b = 0; b < NV; ++b)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[b][i] = o[b][i] * c1 + slot[(b * 16 + i) * KA_WAVE + lane] * c2;
            l = l * c1 + l2 * c2;
            m = m_new;
        }
        __syncthreads();
    }
    if (wave != 0 || !live) return;
    if (n_splits > 1) {
        float* pp = partial + (((size_t)tok * H + head) * n_splits + split) * (hdv + 2);
#pragma unroll
        for (int b = 0; b < NV; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int ch = v0 + b * 32 + (i / 4) * 8 + half * 4 + i % 4;
                if (ch < hdv) pp[ch] = o[b][i];
            }
        if (v0 == 0 && half == 0) {
            pp[hdv] = m;
            pp[hdv + 1] = l;
        }
        return;
    }
    if (has_sink) {
        const float m_new = fmaxf(m, sink2);
        const float c = __builtin_amdgcn_exp2f(m - m_new);
        l = l * c + __builtin_amdgcn_exp2f(sink2 - m_new);
#pragma unroll
        for (int b = 0; b < NV; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[b][i] *= c;
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    // register i of block b: channel v0 + b * 32 + (i / 4) * 8 + half * 4 + i % 4 of the lane's column
    const size_t out_at = (size_t)tok * out_row_stride + (size_t)head * hdv;
    bf16_t* op = out + out_at;
    if (gate && gate_per_head) {
        const float y = 1.0f / (1.0f + __expf(-(float)gate[(size_t)tok * gate_row_stride + head]));
#pragma unroll
        for (int b = 0; b < NV; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[b][i] *= y;
    } else if (gate) {
        // an output gate: every channel times the sigmoid of the gate's pre-activation of the same token and channel
        const bf16_t* gp = gate + (size_t)tok * gate_row_stride + (size_t)head * hdv;
#pragma unroll
        for (int b = 0; b < NV; ++b)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int ch = v0 + b * 32 + (i / 4) * 8 + half * 4 + i % 4;
                if (ch < hdv) o[b][i] *= 1.0f / (1.0f + __expf(-(float)gp[ch]));
            }
    }
    if (out_f32) {
        float* fp = reinterpret_cast<float*>(out) + out_at;
#pragma unroll
        for (int b = 0; b < NV; ++b)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int ch = v0 + b * 32 + g4 * 8 + half * 4;
                if (ch + 3 < hdv) {
                    float4 y = make_float4(o[b][g4 * 4] * inv, o[b][g4 * 4 + 1] * inv, o[b][g4 * 4 + 2] * inv, o[b][g4 * 4 + 3] * inv);
                    *reinterpret_cast<float4*>(fp + ch) = y;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (ch + e < hdv) fp[ch + e] = o[b][g4 * 4 + e] * inv;
                }
            }
        return;
    }
#pragma unroll
    for (int b = 0; b < NV; ++b)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
            const int ch = v0 + b * 32 + g4 * 8 + half * 4;
            if (ch + 3 < hdv) {
                ab_bf16x4 y;
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = (bf16_t)(o[b][g4 * 4 + e] * inv);
                *reinterpret_cast<ab_bf16x4*>(op + ch) = y;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (ch + e < hdv) op[ch + e] = (bf16_t)(o[b][g4 * 4 + e] * inv);
            }
        }
}

// Merges the partial results of a decode step whose rows' keys were split over workgroups: a wave per (token, head).
__global__ void __launch_bounds__(KA_WAVE)
attn_biased_finish_kernel(const float* __restrict__ partial, int n_splits, int H, int hdv, void* __restrict__ out,
                          long out_row_stride, int out_f32, int has_sink, float sink_score, const float* __restrict__ sinks,
                          const bf16_t* __restrict__ gate, long gate_row_stride, int gate_per_head) {
    const int tok = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* pp = partial + ((size_t)tok * H + head) * n_splits * (hdv + 2);
    const float sink2 = (sinks ? sinks[head] : sink_score) * AB_LOG2E;
    float top = has_sink ? sink2 : -INFINITY;
    for (int s = 0; s < n_splits; ++s) top = fmaxf(top, pp[(size_t)s * (hdv + 2) + hdv]);
    float total = has_sink ? __builtin_amdgcn_exp2f(sink2 - top) : 0.f;
    for (int s = 0; s < n_splits; ++s) {
        const float ms = pp[(size_t)s * (hdv + 2) + hdv], ls = pp[(size_t)s * (hdv + 2) + hdv + 1];
        if (ls > 0.f) total += ls * __builtin_amdgcn_exp2f(ms - top);
    }
    const float inv = total > 0.f ? 1.0f / total : 0.f;
    const size_t out_at = (size_t)tok * out_row_stride + (size_t)head * hdv;
    for (int ch = lane; ch < hdv; ch += KA_WAVE) {
        float acc = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const float ls = pp[(size_t)s * (hdv + 2) + hdv + 1];
            // (a split that saw no key left nothing to add, and its outputs may be anything)
            if (ls > 0.f) acc += pp[(size_t)s * (hdv + 2) + ch] * __builtin_amdgcn_exp2f(pp[(size_t)s * (hdv + 2) + hdv] - top);
        }
        float y = acc * inv;
        if (gate) y *= 1.0f / (1.0f + __expf(-(float)gate[(size_t)tok * gate_row_stride + (gate_per_head ? (size_t)head : (size_t)head * hdv + ch)]));
        if (out_f32) reinterpret_cast<float*>(out)[out_at + ch] = y;
        else reinterpret_cast<bf16_t*>(out)[out_at + ch] = (bf16_t)y;
    }
}

static bool ab_sizes_covered(int hd, int hdv) {
    const int nk = hd / 16, nv = (hdv + 31) / 32;
    return hd % 16 == 0 && hdv % 4 == 0 && nk >= 2 && nk <= 8 && nv >= 1 && nv <= 4;
}

// The wide form: any head size in steps of 16 up to AB_WIDE_MAX_HD channels, any value size in steps of 4.
constexpr int AB_WIDE_MAX_HD = 1024;
static bool ab_sizes_covered_wide(int hd, int hdv) {
    return hd % 16 == 0 && hd >= 32 && hd <= AB_WIDE_MAX_HD && hdv % 4 == 0 && hdv >= 4;
}

// Whether the kernel covers these sizes: query/key heads of 32 to 1,024 channels in steps of 16, value heads in steps
// of 4, pages of 16 (up to 128 channels of either with queries in registers, beyond that in the wide form).
KA_API int ka_attention_biased_supported(int hd, int hdv, int page_size) {
    return page_size == AB_PAGE && (ab_sizes_covered(hd, hdv) || ab_sizes_covered_wide(hd, hdv)) ? 1 : 0;
}

KA_API int ka_attention_biased_query_block() { return AB_COLS; }

// n_blocks > 0: a step with blocks of queries (qblk_row, qblk_tok; cu_q); n_blocks == 0: a decode step of n tokens,
// one per row. waves: 4 or 8 per workgroup.
KA_API int ka_attention_biased_bf16(const void* q, long q_row_stride, const void* k_cache, const void* v_cache,
                                    const int* block_table, int max_pages, const int* qblk_row, const int* qblk_tok,
                                    int n_blocks, const int* cu_q, const int* token_row, const int* kv_lo,
                                    const int* kv_hi, const int* positions, const float* slopes, void* out,
                                    long out_row_stride, float scale, int n, int H, int Hkv, int hd, int hdv,
                                    int page_size, int waves, int has_sink, float sink_score, const float* bias_table,
                                    int bias_len, const void* gate, long gate_row_stride, const float* sinks, int keep_first,
                                    int maps, int values_in_keys, int out_f32, int n_splits, float* partial,
                                    float softcap, int gate_per_head, hipStream_t stream) {
    const char* who = "ka_attention_biased_bf16";
    KA_CHECK(softcap >= 0.f, "%s: a cap on the scores must be positive", who);
    KA_CHECK(n >= 0 && n_blocks >= 0 && H > 0 && Hkv > 0 && H % Hkv == 0, "%s: bad sizes", who);
    const bool wide = !ab_sizes_covered(hd, hdv);
    KA_CHECK(page_size == AB_PAGE && (!wide || ab_sizes_covered_wide(hd, hdv)), "%s: head sizes %d / %d or page size %d not covered", who, hd, hdv, page_size);
    KA_CHECK(max_pages > 0, "%s: bad table width %d", who, max_pages);
    KA_CHECK(waves == 4 || waves == 8, "%s: %d waves", who, waves);
    KA_CHECK((uintptr_t)q % 16 == 0 && q_row_stride % 8 == 0 && (uintptr_t)k_cache % 16 == 0,
             "%s: operands must be 16-byte aligned", who);
    KA_CHECK((uintptr_t)out % (out_f32 ? 16 : 8) == 0 && out_row_stride % 4 == 0, "%s: output rows must be aligned to four values", who);
    KA_CHECK(maps >= 1 && H % maps == 0 && Hkv % maps == 0 && keep_first >= 0, "%s: %d maps do not divide the heads %d and %d", who, maps, H, Hkv);
    KA_CHECK(!values_in_keys || (hdv <= hd && maps == 1), "%s: values inside keys of %d channels cannot have %d", who, hd, hdv);
    KA_CHECK(sinks == nullptr || has_sink, "%s: sink scores without a sink", who);
    KA_CHECK(!out_f32 || gate == nullptr, "%s: the output gate goes with bf16 outputs", who);
    KA_CHECK(values_in_keys || (uintptr_t)v_cache % 16 == 0, "%s: operands must be 16-byte aligned", who);
    KA_CHECK(slopes == nullptr || positions != nullptr, "%s: slopes need the queries' positions", who);
    KA_CHECK(bias_table == nullptr || (positions != nullptr && bias_len > 0), "%s: a distance table needs the queries' positions", who);
    KA_CHECK(n_blocks == 0 || (qblk_row && qblk_tok && cu_q), "%s: blocks of queries need their lists", who);
    KA_CHECK(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || (n_blocks == 0 && partial != nullptr)),
             "%s: %d splits (keys are split in decode steps only, and need room for the partial results)", who, n_splits);
    if (n == 0) return 0;
    const int G = H / Hkv;
    int heads_per_block = 1;
    dim3 grid;
    if (n_blocks > 0) {
        grid = dim3(H, n_blocks);
    } else {
        // (with a single query head per kv head the columns hold one query: heads_per_block 1 would mean blocks)
        heads_per_block = G < 2 ? 2 : (G > AB_COLS ? AB_COLS : G);
        grid = dim3(Hkv * ((G + heads_per_block - 1) / heads_per_block) * n_splits, n);
        KA_CHECK(n <= 65535, "%s: too many decode rows %d", who, n);
    }
    KA_CHECK(grid.y <= 65535, "%s: too many blocks %d", who, (int)grid.y);
    const int nk = wide ? 0 : hd / 16, nv = wide ? 4 : (hdv + 31) / 32;
    if (wide) grid.z = (hdv + 127) / 128;
    // the merge area of the waves and, in the wide form, the queries of the 32 columns
    const size_t lds = (size_t)(waves / 2) * (16 * nv + 2) * KA_WAVE * sizeof(float) + (wide ? (size_t)hd * 32 * sizeof(bf16_t) : 0);
#define AB_LAUNCH(NK, NV)                                                                                                  \
    if (nk == NK && nv == NV) {                                                                                            \
        static bool sized = false;                                                                                         \
        if (!sized) {                                                                                                      \
            (void)hipFuncSetAttribute((const void*)attn_biased_kernel<NK, NV>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); \
            sized = true;                                                                                                  \
        }                                                                                                                  \
        hipLaunchKernelGGL((attn_biased_kernel<NK, NV>), grid, dim3(KA_WAVE * waves), lds, stream, (const bf16_t*)q,       \
                           q_row_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, qblk_row, \
                           qblk_tok, cu_q, token_row, kv_lo, kv_hi, positions, slopes, (bf16_t*)out, out_row_stride, scale, \
                           H, Hkv, hdv, heads_per_block, has_sink, sink_score, bias_table, bias_len, (const bf16_t*)gate, \
                           gate_row_stride, sinks, keep_first, maps, values_in_keys, out_f32, hd, n_splits, partial, softcap, gate_per_head); \
    }
#define AB_LAUNCH_NK(NK) AB_LAUNCH(NK, 1) AB_LAUNCH(NK, 2) AB_LAUNCH(NK, 3) AB_LAUNCH(NK, 4)
    AB_LAUNCH_NK(2) AB_LAUNCH_NK(3) AB_LAUNCH_NK(4) AB_LAUNCH_NK(5) AB_LAUNCH_NK(6) AB_LAUNCH_NK(7) AB_LAUNCH_NK(8)
    AB_LAUNCH(0, 4)
#undef AB_LAUNCH_NK
#undef AB_LAUNCH
    KA_LAUNCH_CHECK();
    if (n_splits > 1) {
        KA_CHECK(H <= 65535, "%s: too many heads %d", who, H);
        hipLaunchKernelGGL(attn_biased_finish_kernel, dim3(n, H), dim3(KA_WAVE), 0, stream, partial, n_splits, H, hdv, out,
                           out_row_stride, out_f32, has_sink, sink_score, sinks, (const bf16_t*)gate, gate_row_stride, gate_per_head);
        KA_LAUNCH_CHECK();
    }
    return 0;
}
