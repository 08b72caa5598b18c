// Generic paged attention: one wavefront per (token, query head), any head size up
// to 1024, any page size, fp32 or bf16 storage, all arithmetic in fp32.
//
// Every token t of the packed batch belongs to request row token_row[t] and sees
// the cached keys at positions [kv_lo[t], kv_hi[t]) of that row (kv_lo optional,
// default 0). A causal token at position p has kv_hi = p + 1; a token inside a
// bidirectional block has kv_hi = end of its block; a window of w has
// kv_lo = max(0, p + 1 - w). The keys of this step are already in the cache.
// Key position k of row r lies at page block_table[r, k / page_size], offset
// k % page_size; key cache [pages, Hkv, page_size, hd], value cache [pages, Hkv, hdv, page_size]:
// values may have another size than queries and keys (hdv channels; the output is [n, H hdv]).
//
// Two optional terms of the scores, for mixers that encode order by distance instead of by a
// rotation, and that let a query attend to nothing:
//  * slopes (fp32 [H]) with positions (int32 [n], the place of every query in its row): the score
//    of query position i against key position j is lowered by slopes[h] * (i - j);
//  * a distance table (fp32 [H, bias_len]) with positions: the score of query position i against key position j is
//    raised by table[h, min(i - j, bias_len - 1)] (a learned bias per head and distance, constant from some distance on);
//  * an output gate (rows of the activation type, [n, H hdv] with a row stride of their own): the output is multiplied
//    element by element by the sigmoid of it;
//  * a sink: one more term exp(sink_score) in the softmax's denominator that carries no value
//    (has_sink != 0). The running maximum and sum then start from that term instead of from nothing.
//    `sinks` (fp32 [H]) gives every head a score of its own for that term;
//  * kept first keys: a query also sees the keys [0, min(keep_first, kv_lo)) of its row, before its window;
//  * several maps per head (maps > 1): query heads and key heads come in groups of `maps` neighbours, map m of a
//    query head reads map m of its key head, and all maps of a key head share one value head: H and Hkv count maps,
//    the value cache has Hkv / maps heads;
//  * values inside the keys (values_in_keys != 0): the value of a key is the first hdv channels of its key row
//    (a cache of latents that are both); v_cache is then not read;
//  * out_f32 != 0: the output is written as fp32 whatever the type of queries and cache;
//  * softcap > 0: the scaled score passes through softcap * tanh(score / softcap) before any bias and the softmax;
//  * gate_per_head != 0: the gate holds one number per head ([n, H]) instead of one per channel.
#include "ka_common.h"

constexpr int ATT_MAX_HD = 1024;

// Four neighbouring elements with one load (the address must be a multiple of 4 elements).
template <typename T>
__device__ __forceinline__ void att_load4(const T* p, float v[4]) {
    typedef __attribute__((ext_vector_type(4))) T vec4;
    const vec4 x = *reinterpret_cast<const vec4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ka_to_float(x[i]);
}

template <typename T>
__global__ void __launch_bounds__(KA_WAVE)
attention_generic_kernel(const T* __restrict__ q, long q_row_stride, const T* __restrict__ k_cache,
                         const T* __restrict__ v_cache, const int* __restrict__ block_table,
                         int max_pages, const int* __restrict__ token_row,
                         const int* __restrict__ kv_lo, const int* __restrict__ kv_hi,
                         T* __restrict__ out, long out_row_stride, float scale, int H, int Hkv,
                         int hd, int hdv, int page_size, const int* __restrict__ positions,
                         const float* __restrict__ slopes, int has_sink, float sink_score,
                         const float* __restrict__ bias_table, int bias_len, const T* __restrict__ gate,
                         long gate_row_stride, const float* __restrict__ sinks, int keep_first, int maps,
                         int values_in_keys, int out_f32, float softcap, int gate_per_head) {
    __shared__ float qs[ATT_MAX_HD];
    __shared__ float ps[KA_WAVE];
    __shared__ long offs[KA_WAVE];   // value cache offset of channel 0 of each key of the chunk
    int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    // (maps == 1: query head h reads kv head h / (H / Hkv), keys and values alike)
    const int vh = h / maps / (H / Hkv);
    const int kvh = vh * maps + h % maps;
    const int Hv = Hkv / maps;
    int row = token_row[t];
    int lo = kv_lo ? kv_lo[t] : 0, hi = kv_hi[t];
    const T* qp = q + (size_t)t * q_row_stride + (size_t)h * hd;
    for (int d = lane; d < hd; d += KA_WAVE) qs[d] = ka_to_float(qp[d]) * scale;
    const float slope = slopes ? slopes[h] : 0.f;
    const int place = (slopes || bias_table) ? positions[t] : 0;
    const float* bias_row = bias_table ? bias_table + (size_t)h * bias_len : nullptr;
    __syncthreads();
    const int* bt = block_table + (size_t)row * max_pages;
    const bool k_vectors = hd % 4 == 0 && reinterpret_cast<uintptr_t>(k_cache) % (4 * sizeof(T)) == 0;
    const bool v_vectors = page_size % 4 == 0 && reinterpret_cast<uintptr_t>(v_cache) % (4 * sizeof(T)) == 0;
    if (sinks) sink_score = sinks[h];
    float m = has_sink ? sink_score : -INFINITY, l = has_sink ? 1.f : 0.f;
    float o[ATT_MAX_HD / KA_WAVE];
#pragma unroll
    for (int i = 0; i < ATT_MAX_HD / KA_WAVE; ++i) o[i] = 0.f;
    const int kept = min(keep_first, lo);            // keys [0, kept) before the window, then [lo, hi)
    for (int part = kept > 0 ? 0 : 1; part < 2; ++part)
    for (int base = part ? lo : 0, hi_here = part ? hi : kept; base < hi_here; base += KA_WAVE) {
        const int hi = hi_here;
        int key = base + lane;
        bool valid = key < hi;
        float s = -INFINITY;
        long off = 0;
        if (valid) {
            int page = bt[key / page_size];
            const T* kp = k_cache + (((long)page * Hkv + kvh) * page_size + key % page_size) * hd;
            off = values_in_keys ? (long)(kp - k_cache) : ((long)page * Hv + vh) * hdv * page_size + key % page_size;
            float acc = 0.f;
            if (k_vectors) {
                // four channels with one load, added in the same order as one by one
                for (int d = 0; d < hd; d += 4) {
                    float k4[4];
                    att_load4(kp + d, k4);
#pragma unroll
                    for (int u = 0; u < 4; ++u) acc = fmaf(qs[d + u], k4[u], acc);
                }
            } else {
                for (int d = 0; d < hd; ++d) acc = fmaf(qs[d], ka_to_float(kp[d]), acc);
            }
            if (softcap > 0.f) acc = softcap * tanhf(acc / softcap);
            s = slopes ? acc - slope * (float)(place - key) : acc;
            if (bias_row) s += bias_row[min(max(place - key, 0), bias_len - 1)];
        }
        float m_new = fmaxf(m, ka_wave_max(s));
        float corr = expf(m - m_new);  // m = -inf at the first chunk gives 0
        float p = valid ? expf(s - m_new) : 0.f;
        l = l * corr + ka_wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        offs[lane] = off;
        __syncthreads();
        int count = min(KA_WAVE, hi - base);
#pragma unroll
        for (int i = 0; i < ATT_MAX_HD / KA_WAVE; ++i) {
            int d = lane + i * KA_WAVE;
            if (d < hdv) {
                float acc = o[i] * corr;
                const T* vd = values_in_keys ? k_cache + d : v_cache + (long)d * page_size;
                int j = 0;
                // A chunk that starts on a multiple of four keys: every four keys from there lie in
                // one page, their values side by side in the cache: one load, added in the same
                // order as one by one.
                if (v_vectors && !values_in_keys && (base & 3) == 0) {
                    for (; j + 3 < count; j += 4) {
                        float v4[4];
                        att_load4(vd + offs[j], v4);
#pragma unroll
                        for (int u = 0; u < 4; ++u) acc = fmaf(ps[j + u], v4[u], acc);
                    }
                }
                for (; j < count; ++j) acc = fmaf(ps[j], ka_to_float(vd[offs[j]]), acc);
                o[i] = acc;
            }
        }
    }
    float inv = l > 0.f ? 1.0f / l : 0.f;
    const size_t out_at = (size_t)t * out_row_stride + (size_t)h * hdv;
    const float head_gate = gate && gate_per_head ? 1.0f / (1.0f + expf(-ka_to_float(gate[(size_t)t * gate_row_stride + h]))) : 1.f;
#pragma unroll
    for (int i = 0; i < ATT_MAX_HD / KA_WAVE; ++i) {
        int d = lane + i * KA_WAVE;
        if (d < hdv) {
            float y = o[i] * inv * head_gate;
            // (an output gate: the head's channels times the sigmoid of the gate's pre-activations of the same token)
            if (gate && !gate_per_head) y *= 1.0f / (1.0f + expf(-ka_to_float(gate[(size_t)t * gate_row_stride + (size_t)h * hdv + d])));
            if (out_f32) reinterpret_cast<float*>(out)[out_at + d] = y;
            else out[out_at + d] = ka_from_float<T>(y);
        }
    }
}

KA_API int ka_attention_generic(const void* q, int dtype, long q_row_stride, const void* k_cache,
                                const void* v_cache, const int* block_table, int max_pages,
                                const int* token_row, const int* kv_lo, const int* kv_hi, void* out,
                                long out_row_stride, float scale, int n, int H, int Hkv, int hd,
                                int page_size, int hdv, const int* positions, const float* slopes,
                                int has_sink, float sink_score, const float* bias_table, int bias_len,
                                const void* gate, long gate_row_stride, const float* sinks, int keep_first, int maps,
                                int values_in_keys, int out_f32, float softcap, int gate_per_head, hipStream_t stream) {
    KA_CHECK(softcap >= 0.f, "ka_attention_generic: a cap on the scores must be positive");
    KA_CHECK(maps >= 1 && H % maps == 0 && Hkv % maps == 0 && keep_first >= 0, "ka_attention_generic: %d maps do not divide the heads %d and %d", maps, H, Hkv);
    KA_CHECK(!values_in_keys || hdv <= hd, "ka_attention_generic: values inside keys of %d channels cannot have %d", hd, hdv);
    KA_CHECK(sinks == nullptr || has_sink, "ka_attention_generic: sink scores without a sink");
    KA_CHECK(bias_table == nullptr || (positions != nullptr && bias_len > 0), "ka_attention_generic: a distance table needs the queries' positions");
    KA_CHECK(n >= 0 && H > 0 && Hkv > 0 && hd > 0 && hdv > 0, "ka_attention_generic: bad sizes");
    KA_CHECK(hdv <= ATT_MAX_HD, "ka_attention_generic: value size %d above %d", hdv, ATT_MAX_HD);
    KA_CHECK(slopes == nullptr || positions != nullptr, "ka_attention_generic: slopes need the queries' positions");
    KA_CHECK(H % Hkv == 0, "ka_attention_generic: %d query heads do not divide into %d kv heads", H, Hkv);
    KA_CHECK(hd <= ATT_MAX_HD, "ka_attention_generic: head size %d above %d", hd, ATT_MAX_HD);
    KA_CHECK(H <= 65535, "ka_attention_generic: too many heads %d", H);
    KA_CHECK(page_size > 0 && max_pages > 0, "ka_attention_generic: bad paging %d %d", page_size, max_pages);
    if (n == 0) return 0;
    dim3 grid(n, H), block(KA_WAVE);
    if (dtype == KA_F32)
        hipLaunchKernelGGL(attention_generic_kernel<float>, grid, block, 0, stream, (const float*)q, q_row_stride,
                           (const float*)k_cache, (const float*)v_cache, block_table, max_pages, token_row, kv_lo,
                           kv_hi, (float*)out, out_row_stride, scale, H, Hkv, hd, hdv, page_size, positions, slopes, has_sink,
                           sink_score, bias_table, bias_len, (const float*)gate, gate_row_stride, sinks, keep_first, maps, values_in_keys, out_f32, softcap, gate_per_head);
    else if (dtype == KA_BF16)
        hipLaunchKernelGGL(attention_generic_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)q, q_row_stride,
                           (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, token_row, kv_lo,
                           kv_hi, (bf16_t*)out, out_row_stride, scale, H, Hkv, hd, hdv, page_size, positions, slopes, has_sink,
                           sink_score, bias_table, bias_len, (const bf16_t*)gate, gate_row_stride, sinks, keep_first, maps, values_in_keys, out_f32, softcap, gate_per_head);
    else
        KA_CHECK(false, "ka_attention_generic: unsupported dtype %d", dtype);
    KA_LAUNCH_CHECK();
    return 0;
}
