// Kernels of parts that carry something from one step of a sequence to the next besides keys and values, and of
// mixers whose keys are latents: an embedding of token pairs (the token before is state), a short causal convolution
// over time fused with rotation and cache write (its last inputs are state), the combination of several softmax maps
// of a head, the preparation of latent queries and keys, and a gated pair with clamps. fp32 or bf16 storage, all
// arithmetic in fp32.
#include "ka_common.h"

constexpr int SP_THREADS = 256;

// A token id as the step carries it -> the id itself: -1 stays (its embedding was given), ids[t] <= -2 names an entry of
// `pending` (a token that sampling left on the device); anything outside the vocabulary becomes -1.
__device__ __forceinline__ int sp_token(int id, const int* __restrict__ pending, int n_pending, int vocab) {
    if (id <= -2) {
        const int at = -2 - id;
        if (!pending || at >= n_pending) return -1;
        id = pending[at];
    }
    return (unsigned)id < (unsigned)vocab ? id : -1;
}

// ----------------------------------------------------------------------------
// Pair embedding: x[t] += table[(prev * mul_prev + cur * mul_cur) mod buckets], and table[buckets] for the token at
// place 0 of its sequence. The token before the first of a row's tokens is last_token[slot of the row], which the
// second kernel stores after the first has read it (two launches: the first token of a row reads what its last writes).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(SP_THREADS)
pair_embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, const int* __restrict__ pending, int n_pending,
                  int vocab, const int* __restrict__ positions, const int* __restrict__ token_row, const int* __restrict__ cu_q,
                  const int* __restrict__ row_slot, const int* __restrict__ last_token, int buckets, long long mul_prev,
                  long long mul_cur, float* __restrict__ x, int dim) {
    const int t = blockIdx.x;
    const int cur = sp_token(ids[t], pending, n_pending, vocab);
    if (cur < 0) return;
    long long row;
    if (positions[t] == 0) {
        row = buckets;
    } else {
        const int r = token_row[t];
        int prev;
        if (t > cu_q[r]) {
            prev = sp_token(ids[t - 1], pending, n_pending, vocab);
        } else {
            const int slot = row_slot[r];
            if (slot < 0) return;
            prev = last_token[slot];
        }
        if (prev < 0) return;
        row = ((long long)prev * mul_prev + (long long)cur * mul_cur) % (long long)buckets;
        if (row < 0) row += buckets;
    }
    const T* src = table + (size_t)row * dim;
    float* dst = x + (size_t)t * dim;
    for (int d = threadIdx.x; d < dim; d += SP_THREADS) dst[d] += ka_to_float(src[d]);
}

__global__ void last_token_kernel(const int* __restrict__ ids, const int* __restrict__ pending, int n_pending, int vocab,
                                  const int* __restrict__ cu_q, const int* __restrict__ row_slot, int* __restrict__ last_token,
                                  int n_rows) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= n_rows) return;
    const int slot = row_slot[r];
    if (slot < 0 || cu_q[r + 1] <= cu_q[r]) return;
    last_token[slot] = sp_token(ids[cu_q[r + 1] - 1], pending, n_pending, vocab);
}

KA_API int ka_pair_embed(const void* table, int table_dtype, const int* ids, const int* pending, int n_pending, int vocab,
                         const int* positions, const int* token_row, const int* cu_q, const int* row_slot, int* last_token,
                         int buckets, long mul_prev, long mul_cur, float* x, int n, int n_rows, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && n_rows >= 0 && dim > 0 && buckets > 0 && vocab > 0, "ka_pair_embed: bad sizes");
    KA_CHECK(table_dtype == KA_F32 || table_dtype == KA_BF16, "ka_pair_embed: unsupported table dtype %d", table_dtype);
    if (n == 0) return 0;
    if (table_dtype == KA_F32)
        hipLaunchKernelGGL(pair_embed_kernel<float>, dim3(n), dim3(SP_THREADS), 0, stream, (const float*)table, ids, pending, n_pending,
                           vocab, positions, token_row, cu_q, row_slot, last_token, buckets, (long long)mul_prev, (long long)mul_cur, x, dim);
    else
        hipLaunchKernelGGL(pair_embed_kernel<bf16_t>, dim3(n), dim3(SP_THREADS), 0, stream, (const bf16_t*)table, ids, pending, n_pending,
                           vocab, positions, token_row, cu_q, row_slot, last_token, buckets, (long long)mul_prev, (long long)mul_cur, x, dim);
    KA_LAUNCH_CHECK();
    if (n_rows > 0) {
        hipLaunchKernelGGL(last_token_kernel, dim3(ka_cdiv(n_rows, 64)), dim3(64), 0, stream, ids, pending, n_pending, vocab, cu_q,
                           row_slot, last_token, n_rows);
        KA_LAUNCH_CHECK();
    }
    return 0;
}

// ----------------------------------------------------------------------------
// Short causal convolution over time on every channel of projected queries, keys and values, then the rotation of
// queries and keys, then the cache write: one pass over the rows `u` [n, Cq | Ck | Cv] (Cq = Hq hd, Ck = Hk hd, Cv = Hv hdv).
//   y_t[c] = sum_j taps[c, j] * u_(t - K + 1 + j)[c]
// where inputs before the first token of this step come from `state` [slots + 1, K - 1, C] fp32 (the last K - 1 projected
// rows of the sequence, zero for a new one) and K = 0 means no convolution. Rotation of the first `rot` channels of every
// query and key head by place * freqs[i] (interleaved 1: channels 2i, 2i + 1; 0: i, i + rot / 2). Queries go to `q_out`,
// keys into [pages, Hk, page_size, hd], values into [pages, Hv, hdv, page_size]; a negative slot caches nothing.
// The second kernel then moves the state on (it reads `u`, which the first leaves as it was).
// ----------------------------------------------------------------------------
struct ConvArgs {
    const void* u;
    long u_stride;
    const float* taps;
    float* state;
    int K, C;
    const int* cu_q;
    const int* row_slot;
    const int* token_row;
    const int* positions;
    const int* slots;
    void* q_out;
    long q_stride;
    void* k_cache;
    void* v_cache;
    int Hq, Hk, hd, Hv, hdv, page_size;
    const float* freqs;
    int rot, interleaved;
};

template <typename T>
__device__ __forceinline__ float sp_conv_at(const ConvArgs& a, int t, int local, int slot, int c) {
    const T* u = reinterpret_cast<const T*>(a.u);
    if (a.K <= 0) return ka_to_float(u[(size_t)t * a.u_stride + c]);
    float acc = 0.f;
    for (int j = 0; j < a.K; ++j) {
        const int back = a.K - 1 - j;           // how many places before t
        float v = 0.f;
        if (back <= local) v = ka_to_float(u[(size_t)(t - back) * a.u_stride + c]);
        else if (slot >= 0) v = a.state[((size_t)slot * (a.K - 1) + (local - back + a.K - 1)) * a.C + c];
        acc += a.taps[(size_t)c * a.K + j] * v;
    }
    return acc;
}

constexpr int SP_MAX_ROT = 1024;
constexpr int SP_SPREAD_TOKENS = 128;       // up to this many tokens a step, a token's channels are spread over workgroups

// Grid (tokens, workgroups a token): a token's channels are dealt out over its workgroups (a thread per channel in steps
// of a few tokens, where launches are short and latency counts; one workgroup a token in long steps). The angles of a
// token are the same for every head: a workgroup computes their cosines and sines once, into LDS. Of a rotated pair of
// channels the thread of the first computes both convolutions and writes both results.
template <typename T>
__global__ void __launch_bounds__(SP_THREADS) conv_prepare_kernel(ConvArgs a) {
    __shared__ float cs[SP_MAX_ROT / 2], sn[SP_MAX_ROT / 2];
    const int t = blockIdx.x;
    const int r = a.token_row[t];
    const int local = t - a.cu_q[r];
    const int slot = a.row_slot[r];
    const int Cq = a.Hq * a.hd, Ck = a.Hk * a.hd;
    const float place = (float)a.positions[t];
    const int at = a.slots ? a.slots[t] : -1;
    const int page = at >= 0 ? at / a.page_size : 0, off = at >= 0 ? at % a.page_size : 0;
    const int half = a.rot / 2;
    if (a.freqs) {
        for (int i = threadIdx.x; i < half; i += SP_THREADS) sincosf(place * a.freqs[i], &sn[i], &cs[i]);
        __syncthreads();
    }
    T* q_out = reinterpret_cast<T*>(a.q_out) + (size_t)t * a.q_stride;
    T* k_out = reinterpret_cast<T*>(a.k_cache) + ((size_t)page * a.Hk * a.page_size + off) * a.hd;
    for (int c = blockIdx.y * SP_THREADS + threadIdx.x; c < a.C; c += gridDim.y * SP_THREADS) {
        if (c < Cq + Ck) {
            const int within = c < Cq ? c : c - Cq;
            const int head = within / a.hd, d = within % a.hd;
            T* dst = c < Cq ? q_out + c : (at >= 0 ? k_out + (size_t)head * a.page_size * a.hd + d : nullptr);
            if (a.freqs && d < a.rot) {
                const bool first = a.interleaved ? (d & 1) == 0 : d < half;
                if (!first) continue;                   // (written by the thread of its partner)
                const int step = a.interleaved ? 1 : half;
                const int i = a.interleaved ? d / 2 : d;
                const float y = sp_conv_at<T>(a, t, local, slot, c), other = sp_conv_at<T>(a, t, local, slot, c + step);
                if (dst) {
                    dst[0] = ka_from_float<T>(y * cs[i] - other * sn[i]);
                    dst[step] = ka_from_float<T>(other * cs[i] + y * sn[i]);
                }
            } else if (dst) {
                *dst = ka_from_float<T>(sp_conv_at<T>(a, t, local, slot, c));
            }
        } else if (at >= 0) {
            const int within = c - Cq - Ck;
            const int head = within / a.hdv, d = within % a.hdv;
            reinterpret_cast<T*>(a.v_cache)[(((size_t)page * a.Hv + head) * a.hdv + d) * a.page_size + off] =
                ka_from_float<T>(sp_conv_at<T>(a, t, local, slot, c));
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(SP_THREADS) conv_state_kernel(ConvArgs a) {
    const int r = blockIdx.x;
    const int slot = a.row_slot[r];
    const int first = a.cu_q[r], q = a.cu_q[r + 1] - first;
    if (slot < 0 || q <= 0) return;
    const T* u = reinterpret_cast<const T*>(a.u);
    const int keep = a.K - 1;
    float* st = a.state + (size_t)slot * keep * a.C;
    {
        const int c = blockIdx.y * SP_THREADS + threadIdx.x;
        if (c >= a.C) return;
        // entry s stands for the place s - keep relative to the next step's first token; in rising order an entry is
        // read (s + q) before it is written
        for (int s = 0; s < keep; ++s) {
            const int local = q - keep + s;
            st[(size_t)s * a.C + c] = local >= 0 ? ka_to_float(u[(size_t)(first + local) * a.u_stride + c]) : st[(size_t)(s + q) * a.C + c];
        }
    }
}

KA_API int ka_conv_prepare(const void* u, int dtype, long u_stride, const float* taps, float* state, int K, const int* cu_q,
                           const int* row_slot, const int* token_row, const int* positions, const int* slots, void* q_out,
                           long q_stride, void* k_cache, void* v_cache, int n, int n_rows, int Hq, int Hk, int hd, int Hv, int hdv,
                           int page_size, const float* freqs, int rot, int interleaved, hipStream_t stream) {
    KA_CHECK(n >= 0 && n_rows >= 0 && Hq > 0 && Hk > 0 && hd > 0 && Hv > 0 && hdv > 0 && page_size > 0 && K >= 0, "ka_conv_prepare: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_conv_prepare: unsupported dtype %d", dtype);
    KA_CHECK(K == 0 || taps != nullptr, "ka_conv_prepare: taps missing");
    KA_CHECK(K <= 1 || state != nullptr, "ka_conv_prepare: a convolution of %d taps needs its state", K);
    KA_CHECK(freqs == nullptr || (rot > 0 && rot % 2 == 0 && rot <= hd && rot <= SP_MAX_ROT), "ka_conv_prepare: rotation of %d channels of %d", rot, hd);
    KA_CHECK(slots == nullptr || (k_cache != nullptr && v_cache != nullptr), "ka_conv_prepare: cache tensors missing");
    ConvArgs a;
    a.u = u; a.u_stride = u_stride; a.taps = taps; a.state = state; a.K = K;
    a.C = (Hq + Hk) * hd + Hv * hdv;
    KA_CHECK(u_stride >= a.C && q_stride >= (long)Hq * hd, "ka_conv_prepare: strides too small");
    a.cu_q = cu_q; a.row_slot = row_slot; a.token_row = token_row; a.positions = positions; a.slots = slots;
    a.q_out = q_out; a.q_stride = q_stride; a.k_cache = k_cache; a.v_cache = v_cache;
    a.Hq = Hq; a.Hk = Hk; a.hd = hd; a.Hv = Hv; a.hdv = hdv; a.page_size = page_size;
    a.freqs = freqs; a.rot = freqs ? rot : 0; a.interleaved = interleaved;
    if (n == 0) return 0;
    const int blocks = (a.C + SP_THREADS - 1) / SP_THREADS;
    KA_CHECK(blocks <= 65535, "ka_conv_prepare: too many channels %d", a.C);
    if (dtype == KA_F32) hipLaunchKernelGGL(conv_prepare_kernel<float>, dim3(n, n > SP_SPREAD_TOKENS ? 1 : blocks), dim3(SP_THREADS), 0, stream, a);
    else hipLaunchKernelGGL(conv_prepare_kernel<bf16_t>, dim3(n, n > SP_SPREAD_TOKENS ? 1 : blocks), dim3(SP_THREADS), 0, stream, a);
    KA_LAUNCH_CHECK();
    if (K > 1 && n_rows > 0) {
        if (dtype == KA_F32) hipLaunchKernelGGL(conv_state_kernel<float>, dim3(n_rows, blocks), dim3(SP_THREADS), 0, stream, a);
        else hipLaunchKernelGGL(conv_state_kernel<bf16_t>, dim3(n_rows, blocks), dim3(SP_THREADS), 0, stream, a);
        KA_LAUNCH_CHECK();
    }
    return 0;
}

// ----------------------------------------------------------------------------
// Softmax maps of a head combined: with `maps` fp32 [n, H, 2, dv] (two attentions of a head over the same values),
// o = a1 - lambda * a2, then o / sqrt(mean(o^2) + eps) * out_scale over the head's dv values; a wave per head.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(SP_THREADS)
maps_combine_kernel(const float* __restrict__ maps, T* __restrict__ out, long out_stride, int H, int dv, float lambda, float eps,
                    float out_scale) {
    const int t = blockIdx.x;
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    for (int h = wave; h < H; h += SP_THREADS / KA_WAVE) {
        const float* a1 = maps + ((size_t)t * H + h) * 2 * dv;
        const float* a2 = a1 + dv;
        float ss = 0.f;
        for (int d = lane; d < dv; d += KA_WAVE) {
            const float o = a1[d] - lambda * a2[d];
            ss += o * o;
        }
        ss = ka_wave_sum(ss);
        const float r = out_scale / sqrtf(ss / (float)dv + eps);
        T* dst = out + (size_t)t * out_stride + (size_t)h * dv;
        for (int d = lane; d < dv; d += KA_WAVE) dst[d] = ka_from_float<T>((a1[d] - lambda * a2[d]) * r);
    }
}

KA_API int ka_maps_combine(const float* maps, void* out, int out_dtype, long out_stride, int n, int H, int dv, float lambda,
                           float eps, float out_scale, hipStream_t stream) {
    KA_CHECK(n >= 0 && H > 0 && dv > 0 && eps >= 0.f && out_stride >= (long)H * dv, "ka_maps_combine: bad sizes");
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_maps_combine: unsupported dtype %d", out_dtype);
    if (n == 0) return 0;
    if (out_dtype == KA_F32)
        hipLaunchKernelGGL(maps_combine_kernel<float>, dim3(n), dim3(SP_THREADS), 0, stream, maps, (float*)out, out_stride, H, dv, lambda, eps, out_scale);
    else
        hipLaunchKernelGGL(maps_combine_kernel<bf16_t>, dim3(n), dim3(SP_THREADS), 0, stream, maps, (bf16_t*)out, out_stride, H, dv, lambda, eps, out_scale);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Latents of a step made ready. A row of `down` holds, at `q_at`, the query latent (q_rank channels) and, at `kv_at`, the
// key/value latent (rank channels) followed by dr channels of a key part that all heads share. The query latent goes,
// divided by its root mean square and times its gains, to `cq` [n, q_rank]; the key/value latent, normalised the same
// way with gains of its own, and the shared key part, rotated by place * freqs, go side by side into the paged cache
// [pages, 1, page_size, rank + dr] at slots[t] (a negative slot caches nothing).
// ----------------------------------------------------------------------------
__device__ __forceinline__ float sp_block_sum(float v, float* smem) {
    v = ka_wave_sum(v);
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < SP_THREADS / KA_WAVE; ++w) total += smem[w];
    return total;
}

template <typename T>
__global__ void __launch_bounds__(SP_THREADS)
latent_prepare_kernel(const T* __restrict__ down, long stride, int q_at, int q_rank, const float* __restrict__ q_gain,
                      T* __restrict__ cq, int kv_at, int rank, const float* __restrict__ kv_gain, int dr,
                      const float* __restrict__ freqs, int rot, int interleaved, const int* __restrict__ positions,
                      const int* __restrict__ slots, T* __restrict__ cache, float eps) {
    __shared__ float smem[SP_THREADS / KA_WAVE];
    const int t = blockIdx.x;
    const T* row = down + (size_t)t * stride;
    if (q_rank > 0) {
        float s = 0.f;
        for (int d = threadIdx.x; d < q_rank; d += SP_THREADS) { const float v = ka_to_float(row[q_at + d]); s += v * v; }
        const float r = 1.0f / sqrtf(sp_block_sum(s, smem) / (float)q_rank + eps);
        for (int d = threadIdx.x; d < q_rank; d += SP_THREADS)
            cq[(size_t)t * q_rank + d] = ka_from_float<T>(ka_to_float(row[q_at + d]) * r * (q_gain ? q_gain[d] : 1.f));
    }
    const int at = slots ? slots[t] : -1;
    if (at < 0) return;              // (the same for the whole workgroup)
    float s = 0.f;
    for (int d = threadIdx.x; d < rank; d += SP_THREADS) { const float v = ka_to_float(row[kv_at + d]); s += v * v; }
    const float r = 1.0f / sqrtf(sp_block_sum(s, smem) / (float)rank + eps);
    T* dst = cache + (size_t)at * (rank + dr);
    for (int d = threadIdx.x; d < rank; d += SP_THREADS)
        dst[d] = ka_from_float<T>(ka_to_float(row[kv_at + d]) * r * (kv_gain ? kv_gain[d] : 1.f));
    const float place = (float)positions[t];
    const T* kr = row + kv_at + rank;
    for (int d = threadIdx.x; d < dr; d += SP_THREADS) {
        float y = ka_to_float(kr[d]);
        if (freqs && d < rot) {
            const int half = rot / 2;
            const bool first = interleaved ? (d & 1) == 0 : d < half;
            const int partner = interleaved ? (d ^ 1) : (first ? d + half : d - half);
            const int i = interleaved ? d / 2 : (first ? d : d - half);
            const float other = ka_to_float(kr[partner]);
            const float angle = place * freqs[i];
            const float cs = cosf(angle), sn = sinf(angle);
            y = first ? y * cs - other * sn : y * cs + other * sn;
        }
        dst[rank + d] = ka_from_float<T>(y);
    }
}

KA_API int ka_latent_prepare(const void* down, int dtype, long stride, int q_at, int q_rank, const float* q_gain, void* cq,
                             int kv_at, int rank, const float* kv_gain, int dr, const float* freqs, int rot, int interleaved,
                             const int* positions, const int* slots, void* cache, float eps, int n, hipStream_t stream) {
    KA_CHECK(n >= 0 && q_rank >= 0 && rank > 0 && dr >= 0 && eps >= 0.f, "ka_latent_prepare: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_latent_prepare: unsupported dtype %d", dtype);
    KA_CHECK(freqs == nullptr || (rot > 0 && rot % 2 == 0 && rot <= dr && positions != nullptr), "ka_latent_prepare: rotation of %d channels of %d", rot, dr);
    KA_CHECK(slots == nullptr || cache != nullptr, "ka_latent_prepare: cache tensor missing");
    KA_CHECK(stride >= q_at + q_rank && stride >= kv_at + rank + dr, "ka_latent_prepare: row stride too small");
    if (n == 0) return 0;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(latent_prepare_kernel<float>, dim3(n), dim3(SP_THREADS), 0, stream, (const float*)down, stride, q_at, q_rank,
                           q_gain, (float*)cq, kv_at, rank, kv_gain, dr, freqs, freqs ? rot : 0, interleaved, positions, slots, (float*)cache, eps);
    else
        hipLaunchKernelGGL(latent_prepare_kernel<bf16_t>, dim3(n), dim3(SP_THREADS), 0, stream, (const bf16_t*)down, stride, q_at, q_rank,
                           q_gain, (bf16_t*)cq, kv_at, rank, kv_gain, dr, freqs, freqs ? rot : 0, interleaved, positions, slots, (bf16_t*)cache, eps);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The rotated part of every query head copied behind its latent part: src [n, H, d + dr] -> dst [n, H, rank + dr], the
// channels d .. d + dr of a head turned by place * freqs and written at rank .. rank + dr (the first `rank` channels of
// dst are somebody else's).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(SP_THREADS)
rotate_tail_kernel(const T* __restrict__ src, long src_stride, T* __restrict__ dst, long dst_stride, int H, int d, int dr, int rank,
                   const float* __restrict__ freqs, int rot, int interleaved, const int* __restrict__ positions) {
    const int t = blockIdx.x;
    const float place = (float)positions[t];
    for (int e = threadIdx.x; e < H * dr; e += SP_THREADS) {
        const int h = e / dr, c = e % dr;
        const T* q = src + (size_t)t * src_stride + (size_t)h * (d + dr) + d;
        float y = ka_to_float(q[c]);
        if (freqs && c < rot) {
            const int half = rot / 2;
            const bool first = interleaved ? (c & 1) == 0 : c < half;
            const int partner = interleaved ? (c ^ 1) : (first ? c + half : c - half);
            const int i = interleaved ? c / 2 : (first ? c : c - half);
            const float other = ka_to_float(q[partner]);
            const float angle = place * freqs[i];
            const float cs = cosf(angle), sn = sinf(angle);
            y = first ? y * cs - other * sn : y * cs + other * sn;
        }
        dst[(size_t)t * dst_stride + (size_t)h * (rank + dr) + rank + c] = ka_from_float<T>(y);
    }
}

KA_API int ka_rotate_tail(const void* src, int dtype, long src_stride, void* dst, long dst_stride, int n, int H, int d, int dr,
                          int rank, const float* freqs, int rot, int interleaved, const int* positions, hipStream_t stream) {
    KA_CHECK(n >= 0 && H > 0 && d >= 0 && dr > 0 && rank >= 0, "ka_rotate_tail: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_rotate_tail: unsupported dtype %d", dtype);
    KA_CHECK(freqs == nullptr || (rot > 0 && rot % 2 == 0 && rot <= dr), "ka_rotate_tail: rotation of %d channels of %d", rot, dr);
    KA_CHECK(src_stride >= (long)H * (d + dr) && dst_stride >= (long)H * (rank + dr) && positions != nullptr, "ka_rotate_tail: strides too small");
    if (n == 0) return 0;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(rotate_tail_kernel<float>, dim3(n), dim3(SP_THREADS), 0, stream, (const float*)src, src_stride, (float*)dst,
                           dst_stride, H, d, dr, rank, freqs, freqs ? rot : 0, interleaved, positions);
    else
        hipLaunchKernelGGL(rotate_tail_kernel<bf16_t>, dim3(n), dim3(SP_THREADS), 0, stream, (const bf16_t*)src, src_stride, (bf16_t*)dst,
                           dst_stride, H, d, dr, rank, freqs, freqs ? rot : 0, interleaved, positions);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// A gated pair with clamps: for rows whose gate and value sums lie side by side (x[t, 2j], x[t, 2j + 1]),
//   g = min(gate, limit), u = clamp(value, -limit, limit), out[t, j] = g * sigmoid(slope * g) * (u + shift).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(SP_THREADS)
clamped_pairs_kernel(const T* __restrict__ x, long x_stride, T* __restrict__ out, long out_stride, int n_out, float limit, float slope,
                     float shift) {
    const T* xr = x + (size_t)blockIdx.y * x_stride;
    T* orow = out + (size_t)blockIdx.y * out_stride;
    typedef T __attribute__((ext_vector_type(2))) pair_t;
    for (int j = blockIdx.x * SP_THREADS + threadIdx.x; j < n_out; j += gridDim.x * SP_THREADS) {
        const pair_t p = *reinterpret_cast<const pair_t*>(xr + 2 * (size_t)j);
        const float g = fminf(ka_to_float(p[0]), limit);
        const float u = fminf(fmaxf(ka_to_float(p[1]), -limit), limit);
        orow[j] = ka_from_float<T>(g / (1.0f + expf(-slope * g)) * (u + shift));
    }
}

KA_API int ka_clamped_pairs(const void* x, long x_stride, void* out, long out_stride, int dtype, int n, int n_out, float limit,
                            float slope, float shift, hipStream_t stream) {
    KA_CHECK(n >= 0 && n_out > 0 && x_stride >= 2L * n_out && out_stride >= n_out && x_stride % 2 == 0, "ka_clamped_pairs: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_clamped_pairs: unsupported dtype %d", dtype);
    KA_CHECK(n <= 65535, "ka_clamped_pairs: too many rows %d", n);
    KA_CHECK((uintptr_t)x % (dtype == KA_F32 ? 8 : 4) == 0, "ka_clamped_pairs: pairs must be aligned");
    if (n == 0) return 0;
    const int blocks = ka_cdiv(n_out, SP_THREADS * 4) < 1 ? 1 : ka_cdiv(n_out, SP_THREADS * 4);
    const dim3 grid(blocks, n);
    if (dtype == KA_F32)
        hipLaunchKernelGGL(clamped_pairs_kernel<float>, grid, dim3(SP_THREADS), 0, stream, (const float*)x, x_stride, (float*)out, out_stride, n_out, limit, slope, shift);
    else
        hipLaunchKernelGGL(clamped_pairs_kernel<bf16_t>, grid, dim3(SP_THREADS), 0, stream, (const bf16_t*)x, x_stride, (bf16_t*)out, out_stride, n_out, limit, slope, shift);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// x[t] += v for every row of fp32 x [n, dim] (a learned vector that enters the stream at a junction).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void add_vector_kernel(float* __restrict__ x, const T* __restrict__ v, long count, int dim) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) x[i] += ka_to_float(v[i % dim]);
}

KA_API int ka_add_vector(float* x, const void* v, int v_dtype, int n, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0, "ka_add_vector: bad sizes");
    KA_CHECK(v_dtype == KA_F32 || v_dtype == KA_BF16, "ka_add_vector: unsupported dtype %d", v_dtype);
    const long count = (long)n * dim;
    if (count == 0) return 0;
    const unsigned blocks = (unsigned)((count + 255) / 256);
    if (v_dtype == KA_F32) hipLaunchKernelGGL(add_vector_kernel<float>, dim3(blocks), dim3(256), 0, stream, x, (const float*)v, count, dim);
    else hipLaunchKernelGGL(add_vector_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, x, (const bf16_t*)v, count, dim);
    KA_LAUNCH_CHECK();
    return 0;
}
