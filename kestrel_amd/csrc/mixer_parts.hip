// Kernels of mixers that are more than "rotate, cache, attend": a root-mean-square norm, the preparation of
// queries, keys and values of a step in one pass (norm with gains over a head or over the whole projection, a
// rotation from frequencies, a factor on queries that grows with the place, values blended with those of another
// layer, the paged cache write), an output gate, the sum of normalised branches, and a gated matrix memory
// (a recurrent mixer with a state of fixed size per request). fp32 or bf16 storage, all arithmetic in fp32.
#include "ka_common.h"

constexpr int MP_THREADS = 256;
constexpr int MP_WAVES = MP_THREADS / KA_WAVE;

// Sum over the 256 threads of a workgroup, the same bits in every thread; `smem` holds MP_WAVES floats.
__device__ __forceinline__ float mp_block_sum(float v, float* smem) {
    v = ka_wave_sum(v);
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < MP_WAVES; ++w) total += smem[w];
    return total;
}

__device__ __forceinline__ float mp_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

// ----------------------------------------------------------------------------
// Root-mean-square norm: out = x / sqrt(mean(x^2) + eps) * gain over the last axis of fp32 rows (all, or
// those that `rows` names).
// ----------------------------------------------------------------------------
template <typename TOut>
__global__ void __launch_bounds__(MP_THREADS)
rmsnorm_kernel(const float* __restrict__ x, const int* __restrict__ rows, const float* __restrict__ gain, float eps,
               TOut* __restrict__ out, int dim) {
    __shared__ float smem[MP_WAVES];
    const int i = blockIdx.x;
    const float* src = x + (size_t)(rows ? rows[i] : i) * dim;
    TOut* dst = out + (size_t)i * dim;
    float s = 0.f;
    for (int d = threadIdx.x; d < dim; d += MP_THREADS) s += src[d] * src[d];
    const float r = 1.0f / sqrtf(mp_block_sum(s, smem) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += MP_THREADS) dst[d] = ka_from_float<TOut>(src[d] * r * (gain ? gain[d] : 1.f));
}

KA_API int ka_rmsnorm(const float* x, const int* rows, const float* gain, float eps, void* out, int out_dtype, int n,
                      int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && eps >= 0.f, "ka_rmsnorm: bad sizes n=%d dim=%d", n, dim);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_rmsnorm: unsupported out dtype %d", out_dtype);
    if (n == 0) return 0;
    if (out_dtype == KA_F32)
        hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3(n), dim3(MP_THREADS), 0, stream, x, rows, gain, eps, (float*)out, dim);
    else
        hipLaunchKernelGGL(rmsnorm_kernel<bf16_t>, dim3(n), dim3(MP_THREADS), 0, stream, x, rows, gain, eps, (bf16_t*)out, dim);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Queries, keys and values of a step made ready for attention, a workgroup per token, a wave per head in turns.
// Row of `qkv`: [H hd queries | G hd keys | G hdv values]. In this order:
//  * norm (norm_mode 1: every query and key head divided by its root mean square, gains [hd] shared by the
//    heads; 2: all queries of the token by the root mean square over the whole H hd, likewise all keys, gains
//    [H hd] and [G hd]; 0: none); gains optional;
//  * rotation of the first `rot` channels of every head by the angles place * freqs[i], computed here in fp32
//    (interleaved 1: channels 2i and 2i + 1 are a pair, 0: channels i and i + rot / 2); freqs null: none;
//  * queries times 1 + q_coef * ln(floor((place + 1) / q_every) + 1) (q_every 0: no such factor);
//  * values: blend 1 copies them to `v_other` (the values of this layer for later ones), blend 2 replaces them by
//    (1 - lambda) v + lambda v_other with the fp32 scalar at `lambda`;
//  * queries go back in place; keys go into the paged cache [pages, G, page_size, hd] (the row keeps them as projected),
//    values into [pages, G, hdv, page_size] (slots[t] = page * page_size + offset, negative or no slots: nothing is cached);
//  * v_from_k != 0: there are no value columns, the values are the keys as projected (hdv = hd; the row is
//    [H hd | G hd]); G = 0: a row of queries alone (a layer that reads another layer's keys and values).
// ----------------------------------------------------------------------------
struct PrepareArgs {
    void* qkv;
    long row_stride;
    const int* positions;
    const int* slots;
    void* k_cache;
    void* v_cache;
    int H, G, hd, hdv, page_size;
    int norm_mode;
    const float* q_gain;
    const float* k_gain;
    float eps;
    const float* freqs;
    int rot, interleaved;
    float q_coef;
    int q_every;
    int blend;
    void* v_other;
    long v_other_stride;
    const float* lambda;
    int v_from_k;
};

template <typename T>
__global__ void __launch_bounds__(MP_THREADS) qkv_prepare_kernel(PrepareArgs a) {
    extern __shared__ float sm[];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int wave = tid / KA_WAVE, lane = tid % KA_WAVE;
    const int heads = a.H + a.G, half = a.rot / 2, hd = a.hd;
    float* cs = sm;                    // cosines, then sines, of the token's angles
    float* sn = cs + half;
    float* ss = sn + half;             // sum of squares per head
    T* row = reinterpret_cast<T*>(a.qkv) + (size_t)t * a.row_stride;
    const int pos = a.positions ? a.positions[t] : 0;
    if (a.freqs)
        for (int i = tid; i < half; i += MP_THREADS) sincosf((float)pos * a.freqs[i], &sn[i], &cs[i]);
    // a wave per head, in turns
    if (a.norm_mode) {
        for (int h = wave; h < heads; h += MP_WAVES) {
            const T* hp = row + (size_t)h * hd;
            float s = 0.f;
            for (int c = lane; c < hd; c += KA_WAVE) {
                const float x = ka_to_float(hp[c]);
                s += x * x;
            }
            s = ka_wave_sum(s);
            if (lane == 0) ss[h] = s;
        }
    }
    __syncthreads();
    float r_all_q = 1.f, r_all_k = 1.f;
    if (a.norm_mode == 2) {
        float sq = 0.f, sk = 0.f;
        for (int h = 0; h < a.H; ++h) sq += ss[h];
        for (int h = a.H; h < heads; ++h) sk += ss[h];
        r_all_q = 1.0f / sqrtf(sq / (float)(a.H * hd) + a.eps);
        r_all_k = 1.0f / sqrtf(sk / (float)(a.G * hd) + a.eps);
    }
    const float q_factor = a.q_every > 0 ? 1.0f + a.q_coef * logf((float)((pos + 1) / a.q_every + 1)) : 1.0f;
    const long slot = a.slots ? a.slots[t] : -1;
    const long page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
    T* k_cache = reinterpret_cast<T*>(a.k_cache);
    T* v_cache = reinterpret_cast<T*>(a.v_cache);
    for (int h = wave; h < heads; h += MP_WAVES) {
        const bool is_q = h < a.H;
        if (!is_q && slot < 0) continue;            // (a key that is cached nowhere: nobody reads it)
        T* hp = row + (size_t)h * hd;
        // where the head's results go: queries back in place, keys into the cache
        T* dst = is_q ? hp : k_cache + (((size_t)page * a.G + (h - a.H)) * a.page_size + off) * hd;
        float r = 1.f;
        const float* gain = nullptr;
        if (a.norm_mode == 1) {
            r = 1.0f / sqrtf(ss[h] / (float)hd + a.eps);
            gain = is_q ? a.q_gain : a.k_gain;
        } else if (a.norm_mode == 2) {
            r = is_q ? r_all_q : r_all_k;
            gain = is_q ? a.q_gain : a.k_gain;
            if (gain) gain += (size_t)(is_q ? h : h - a.H) * hd;
        }
        const float after = is_q ? q_factor : 1.f;
        // a rotated pair is one lane's: both of its channels are read before either is written
        if (a.freqs) {
            for (int i = lane; i < half; i += KA_WAVE) {
                const int ia = a.interleaved ? 2 * i : i, ib = a.interleaved ? 2 * i + 1 : i + half;
                const float u = ka_to_float(hp[ia]) * r * (gain ? gain[ia] : 1.f);
                const float v = ka_to_float(hp[ib]) * r * (gain ? gain[ib] : 1.f);
                dst[ia] = ka_from_float<T>((u * cs[i] - v * sn[i]) * after);
                dst[ib] = ka_from_float<T>((v * cs[i] + u * sn[i]) * after);
            }
        }
        for (int c = a.rot + lane; c < hd; c += KA_WAVE)
            dst[c] = ka_from_float<T>(ka_to_float(hp[c]) * r * (gain ? gain[c] : 1.f) * after);
    }
    T* vrow = row + (size_t)(a.v_from_k ? a.H : heads) * hd;
    const float lam = a.blend == 2 ? *a.lambda : 0.f;
    T* other = a.blend ? reinterpret_cast<T*>(a.v_other) + (size_t)t * a.v_other_stride : nullptr;
    for (int g = wave; g < a.G; g += MP_WAVES)
        for (int c = lane; c < a.hdv; c += KA_WAVE) {
            const int e = g * a.hdv + c;
            T v = vrow[e];
            if (a.blend == 1) other[e] = v;
            else if (a.blend == 2) v = ka_from_float<T>((1.0f - lam) * ka_to_float(v) + lam * ka_to_float(other[e]));
            if (slot >= 0) v_cache[(((size_t)page * a.G + g) * a.hdv + c) * a.page_size + off] = v;
        }
}

// The same for bf16 rows whose heads are 32, 64 or 128 channels wide: a lane takes eight neighbouring channels with one
// 16-byte load, LPH lanes a head, so that a wave covers 64 / LPH heads at a time and a head's sum of squares meets inside
// its lanes. A rotated pair of neighbours (channels 2i and 2i + 1) lies inside a lane's eight; a pair of halves (i and
// i + rot / 2, rot a multiple of 16) in two lanes of the head, which exchange their numbers. Values in pieces of eight as well.
typedef __attribute__((ext_vector_type(8))) __bf16 mp_bf16x8;
typedef __attribute__((ext_vector_type(4))) float mp_floatx4;

template <int LPH>
__global__ void __launch_bounds__(MP_THREADS) qkv_prepare_wide_kernel(PrepareArgs a) {
    extern __shared__ float sm[];
    constexpr int HD = 8 * LPH, HEADS_A_PASS = MP_THREADS / LPH;
    const int t = blockIdx.x, tid = threadIdx.x;
    const int group = tid / LPH, sub = tid % LPH;
    const int heads = a.H + a.G, half = a.rot / 2;
    float* cs = sm;
    float* sn = cs + half;
    float* ss = sn + half;
    bf16_t* row = reinterpret_cast<bf16_t*>(a.qkv) + (size_t)t * a.row_stride;
    const int pos = a.positions ? a.positions[t] : 0;
    if (a.freqs)
        for (int i = tid; i < half; i += MP_THREADS) sincosf((float)pos * a.freqs[i], &sn[i], &cs[i]);
    if (a.norm_mode) {
        for (int h0 = 0; h0 < heads; h0 += HEADS_A_PASS) {
            const int h = h0 + group;
            float s = 0.f;
            if (h < heads) {
                const mp_bf16x8 x = *reinterpret_cast<const mp_bf16x8*>(row + (size_t)h * HD + sub * 8);
#pragma unroll
                for (int u = 0; u < 8; ++u) s += (float)x[u] * (float)x[u];
            }
            s = ka_lanes_reduce<1, LPH>(s, KaSum{});
            if (h < heads && sub == 0) ss[h] = s;
        }
    }
    __syncthreads();
    float r_all_q = 1.f, r_all_k = 1.f;
    if (a.norm_mode == 2) {
        float sq = 0.f, sk = 0.f;
        for (int h = 0; h < a.H; ++h) sq += ss[h];
        for (int h = a.H; h < heads; ++h) sk += ss[h];
        r_all_q = 1.0f / sqrtf(sq / (float)(a.H * HD) + a.eps);
        r_all_k = 1.0f / sqrtf(sk / (float)(a.G * HD) + a.eps);
    }
    const float q_factor = a.q_every > 0 ? 1.0f + a.q_coef * logf((float)((pos + 1) / a.q_every + 1)) : 1.0f;
    const long slot = a.slots ? a.slots[t] : -1;
    const long page = slot >= 0 ? slot / a.page_size : 0, off = slot >= 0 ? slot % a.page_size : 0;
    bf16_t* k_cache = reinterpret_cast<bf16_t*>(a.k_cache);
    bf16_t* v_cache = reinterpret_cast<bf16_t*>(a.v_cache);
    for (int h = group; h < heads; h += HEADS_A_PASS) {
        const bool is_q = h < a.H;
        if (!is_q && slot < 0) continue;
        bf16_t* hp = row + (size_t)h * HD + sub * 8;
        bf16_t* dst = is_q ? hp : k_cache + (((size_t)page * a.G + (h - a.H)) * a.page_size + off) * HD + sub * 8;
        float r = 1.f;
        const float* gain = nullptr;
        if (a.norm_mode == 1) {
            r = 1.0f / sqrtf(ss[h] / (float)HD + a.eps);
            gain = is_q ? a.q_gain : a.k_gain;
        } else if (a.norm_mode == 2) {
            r = is_q ? r_all_q : r_all_k;
            gain = is_q ? a.q_gain : a.k_gain;
            if (gain) gain += (size_t)(is_q ? h : h - a.H) * HD;
        }
        const float after = is_q ? q_factor : 1.f;
        const mp_bf16x8 x = *reinterpret_cast<const mp_bf16x8*>(hp);
        float y[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) y[u] = (float)x[u] * r;
        if (gain) {
            const mp_floatx4 g0 = *reinterpret_cast<const mp_floatx4*>(gain + sub * 8);
            const mp_floatx4 g1 = *reinterpret_cast<const mp_floatx4*>(gain + sub * 8 + 4);
#pragma unroll
            for (int u = 0; u < 4; ++u) { y[u] *= g0[u]; y[4 + u] *= g1[u]; }
        }
        if (a.freqs && a.interleaved) {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int i = sub * 4 + p;
                if (2 * i < a.rot) {
                    const float u = y[2 * p], v = y[2 * p + 1];
                    y[2 * p] = u * cs[i] - v * sn[i];
                    y[2 * p + 1] = v * cs[i] + u * sn[i];
                }
            }
        } else if (a.freqs) {
            // halves: channel c turns with channel c + rot / 2, which the lane rot / 16 further on holds (rot is a multiple
            // of 16 here): the lanes of a pair exchange their eight numbers
            const int apart = a.rot / 16;
            const bool low = sub < apart, turned = sub < 2 * apart;
            const int partner = (tid % KA_WAVE) + (low ? apart : -apart);
            float other[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) other[u] = __shfl(y[u], turned ? partner : tid % KA_WAVE);
            if (turned) {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int i = (low ? sub : sub - apart) * 8 + u;
                    y[u] = low ? y[u] * cs[i] - other[u] * sn[i] : y[u] * cs[i] + other[u] * sn[i];
                }
            }
        }
        mp_bf16x8 o;
#pragma unroll
        for (int u = 0; u < 8; ++u) o[u] = (bf16_t)(y[u] * after);
        *reinterpret_cast<mp_bf16x8*>(dst) = o;
    }
    bf16_t* vrow = row + (size_t)(a.v_from_k ? a.H : heads) * HD;
    const int pieces = a.hdv / 8;
    const float lam = a.blend == 2 ? *a.lambda : 0.f;
    bf16_t* other = a.blend ? reinterpret_cast<bf16_t*>(a.v_other) + (size_t)t * a.v_other_stride : nullptr;
    for (int e = tid; e < a.G * pieces; e += MP_THREADS) {
        const int g = e / pieces, c0 = (e % pieces) * 8;
        mp_bf16x8 v = *reinterpret_cast<const mp_bf16x8*>(vrow + (size_t)g * a.hdv + c0);
        if (a.blend == 1) {
            *reinterpret_cast<mp_bf16x8*>(other + (size_t)g * a.hdv + c0) = v;
        } else if (a.blend == 2) {
            const mp_bf16x8 w = *reinterpret_cast<const mp_bf16x8*>(other + (size_t)g * a.hdv + c0);
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = (bf16_t)((1.0f - lam) * (float)v[u] + lam * (float)w[u]);
        }
        if (slot >= 0) {
            bf16_t* vp = v_cache + (((size_t)page * a.G + g) * a.hdv + c0) * a.page_size + off;
#pragma unroll
            for (int u = 0; u < 8; ++u) vp[(size_t)u * a.page_size] = v[u];
        }
    }
}

KA_API int ka_qkv_prepare(void* qkv, int dtype, long row_stride, const int* positions, const int* slots, void* k_cache,
                          void* v_cache, int n, int H, int G, int hd, int hdv, int page_size, int norm_mode,
                          const float* q_gain, const float* k_gain, float eps, const float* freqs, int rot, int interleaved,
                          float q_coef, int q_every, int blend, void* v_other, long v_other_stride, const float* lambda,
                          int v_from_k, hipStream_t stream) {
    const char* who = "ka_qkv_prepare";
    KA_CHECK(n >= 0 && H > 0 && G >= 0 && hd > 0 && hdv > 0 && page_size > 0, "%s: bad sizes", who);
    KA_CHECK(!v_from_k || (hdv == hd && blend == 0), "%s: values that are the keys have the keys' size and are not blended", who);
    KA_CHECK(G > 0 || slots == nullptr, "%s: a row of queries alone caches nothing", who);
    KA_CHECK(row_stride >= (long)(H + G) * hd + (v_from_k ? 0 : (long)G * hdv), "%s: row stride %ld too small", who, row_stride);
    KA_CHECK(norm_mode >= 0 && norm_mode <= 2 && eps >= 0.f, "%s: norm mode %d", who, norm_mode);
    KA_CHECK(freqs == nullptr || (rot > 0 && rot <= hd && rot % 2 == 0), "%s: %d rotated channels of %d", who, rot, hd);
    KA_CHECK(freqs == nullptr || positions != nullptr, "%s: a rotation needs the tokens' places", who);
    KA_CHECK(q_every >= 0 && (q_every == 0 || positions != nullptr), "%s: the queries' factor needs the tokens' places", who);
    KA_CHECK(interleaved == 0 || interleaved == 1, "%s: pairing must be 0 (halves) or 1 (interleaved)", who);
    KA_CHECK(blend >= 0 && blend <= 2 && (blend == 0 || (v_other != nullptr && v_other_stride >= (long)G * hdv)),
             "%s: blended values need the other layer's values", who);
    KA_CHECK(blend != 2 || lambda != nullptr, "%s: a blend needs its weight", who);
    KA_CHECK(slots == nullptr || (k_cache != nullptr && v_cache != nullptr), "%s: cache tensors missing", who);
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "%s: unsupported dtype %d", who, dtype);
    if (n == 0) return 0;
    if (freqs == nullptr) rot = 0;
    const size_t lds = ((size_t)(H + G) + rot) * sizeof(float);
    KA_CHECK(lds <= 64 * 1024, "%s: %d heads and %d rotated channels do not fit in LDS", who, H + G, rot);
    PrepareArgs a{qkv, row_stride, positions, slots, k_cache, v_cache, H, G, hd, hdv, page_size, norm_mode, q_gain, k_gain, eps,
                  freqs, rot, interleaved, q_coef, q_every, blend, v_other, v_other_stride, lambda, v_from_k};
    // bf16 heads of 32, 64 or 128 channels, everything 16-byte aligned, pairs of neighbours if rotated: eight channels a lane
    const bool wide = dtype == KA_BF16 && (hd == 32 || hd == 64 || hd == 128) && hdv % 8 == 0 && row_stride % 8 == 0 &&
        (uintptr_t)qkv % 16 == 0 && (freqs == nullptr || interleaved == 1 || rot % 16 == 0) &&
        (blend == 0 || ((uintptr_t)v_other % 16 == 0 && v_other_stride % 8 == 0)) &&
        (uintptr_t)q_gain % 16 == 0 && (uintptr_t)k_gain % 16 == 0 && (slots == nullptr || (uintptr_t)k_cache % 16 == 0);
    if (wide && hd == 32) hipLaunchKernelGGL(qkv_prepare_wide_kernel<4>, dim3(n), dim3(MP_THREADS), lds, stream, a);
    else if (wide && hd == 64) hipLaunchKernelGGL(qkv_prepare_wide_kernel<8>, dim3(n), dim3(MP_THREADS), lds, stream, a);
    else if (wide) hipLaunchKernelGGL(qkv_prepare_wide_kernel<16>, dim3(n), dim3(MP_THREADS), lds, stream, a);
    else if (dtype == KA_F32) hipLaunchKernelGGL(qkv_prepare_kernel<float>, dim3(n), dim3(MP_THREADS), lds, stream, a);
    else hipLaunchKernelGGL(qkv_prepare_kernel<bf16_t>, dim3(n), dim3(MP_THREADS), lds, stream, a);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Output gate: x[t, :] *= sigmoid(gate[t, :]) (both of the activation type, rows with strides of their own).
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(MP_THREADS)
gate_mul_kernel(T* __restrict__ x, long x_stride, const T* __restrict__ gate, long gate_stride, int dim) {
    T* xr = x + (size_t)blockIdx.x * x_stride;
    const T* gr = gate + (size_t)blockIdx.x * gate_stride;
    for (int d = threadIdx.x; d < dim; d += MP_THREADS) xr[d] = ka_from_float<T>(ka_to_float(xr[d]) * mp_sigmoid(ka_to_float(gr[d])));
}

KA_API int ka_gate_mul(void* x, long x_stride, const void* gate, long gate_stride, int dtype, int n, int dim, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && x_stride >= dim && gate_stride >= dim, "ka_gate_mul: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_gate_mul: unsupported dtype %d", dtype);
    if (n == 0) return 0;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(gate_mul_kernel<float>, dim3(n), dim3(MP_THREADS), 0, stream, (float*)x, x_stride, (const float*)gate, gate_stride, dim);
    else
        hipLaunchKernelGGL(gate_mul_kernel<bf16_t>, dim3(n), dim3(MP_THREADS), 0, stream, (bf16_t*)x, x_stride, (const bf16_t*)gate, gate_stride, dim);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The product of a gated pair: out[t, j] = act(x[t, 2j]) * x[t, 2j + 1] for rows whose gate and value sums lie side by
// side (what a plain linear over paired weight rows leaves): the second half of a gated linear whose first half went
// through a kernel that has no such epilogue (the vendor library's). Rows of the activation type.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(MP_THREADS)
gated_pairs_kernel(const T* __restrict__ x, long x_stride, T* __restrict__ out, long out_stride, int n_out, int act) {
    const T* xr = x + (size_t)blockIdx.y * x_stride;
    T* orow = out + (size_t)blockIdx.y * out_stride;
    typedef T __attribute__((ext_vector_type(2))) pair_t;
    for (int j = blockIdx.x * MP_THREADS + threadIdx.x; j < n_out; j += gridDim.x * MP_THREADS) {
        const pair_t p = *reinterpret_cast<const pair_t*>(xr + 2 * (size_t)j);
        const float g = sizeof(T) == 2 ? ka_activate_fast(act, ka_to_float(p[0])) : ka_activate(act, ka_to_float(p[0]));
        orow[j] = ka_from_float<T>(g * ka_to_float(p[1]));
    }
}

KA_API int ka_gated_pairs(const void* x, long x_stride, void* out, long out_stride, int dtype, int n, int n_out, int act,
                          hipStream_t stream) {
    KA_CHECK(n >= 0 && n_out > 0 && x_stride >= 2L * n_out && out_stride >= n_out && x_stride % 2 == 0, "ka_gated_pairs: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_gated_pairs: unsupported dtype %d", dtype);
    KA_CHECK(ka_act_known(act) && !ka_act_gated(act), "ka_gated_pairs: unknown activation %d", act);
    KA_CHECK(n <= 65535, "ka_gated_pairs: too many rows %d", n);
    KA_CHECK((uintptr_t)x % (dtype == KA_F32 ? 8 : 4) == 0, "ka_gated_pairs: pairs must be aligned");
    if (n == 0) return 0;
    const int blocks = ka_cdiv(n_out, MP_THREADS * 4) < 1 ? 1 : ka_cdiv(n_out, MP_THREADS * 4);
    const dim3 grid(blocks, n);
    if (dtype == KA_F32)
        hipLaunchKernelGGL(gated_pairs_kernel<float>, grid, dim3(MP_THREADS), 0, stream, (const float*)x, x_stride, (float*)out, out_stride, n_out, act);
    else
        hipLaunchKernelGGL(gated_pairs_kernel<bf16_t>, grid, dim3(MP_THREADS), 0, stream, (const bf16_t*)x, x_stride, (bf16_t*)out, out_stride, n_out, act);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The sum of normalised branches into the stream: x += ca * rms(a) * gain_a [+ cb * rms(b) * gain_b], every
// branch divided by its own root mean square over the row; all fp32. `rounded` (optional, of type TR): the new rows of the
// stream are left there as well, in the activation type, for a reader that takes them so.
// ----------------------------------------------------------------------------
template <typename TR>
__global__ void __launch_bounds__(MP_THREADS)
branches_sum_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ gain_a, float ca,
                    const float* __restrict__ b, const float* __restrict__ gain_b, float cb, float eps, int dim,
                    TR* __restrict__ rounded) {
    __shared__ float smem[MP_WAVES];
    const size_t at = (size_t)blockIdx.x * dim;
    float sa = 0.f, sb = 0.f;
    for (int d = threadIdx.x; d < dim; d += MP_THREADS) {
        sa += a[at + d] * a[at + d];
        if (b) sb += b[at + d] * b[at + d];
    }
    const float ra = 1.0f / sqrtf(mp_block_sum(sa, smem) / (float)dim + eps);
    const float rb = b ? 1.0f / sqrtf(mp_block_sum(sb, smem) / (float)dim + eps) : 0.f;
    for (int d = threadIdx.x; d < dim; d += MP_THREADS) {
        float y = ca * (a[at + d] * ra * (gain_a ? gain_a[d] : 1.f));
        if (b) y += cb * (b[at + d] * rb * (gain_b ? gain_b[d] : 1.f));
        y += x[at + d];
        x[at + d] = y;
        if (rounded) rounded[at + d] = ka_from_float<TR>(y);
    }
}

KA_API int ka_branches_sum(float* x, const float* a, const float* gain_a, float ca, const float* b, const float* gain_b,
                           float cb, float eps, int n, int dim, void* rounded, int rounded_dtype, hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && eps >= 0.f && a != nullptr, "ka_branches_sum: bad sizes");
    KA_CHECK(rounded == nullptr || rounded_dtype == KA_F32 || rounded_dtype == KA_BF16, "ka_branches_sum: unsupported dtype %d", rounded_dtype);
    if (n == 0) return 0;
    if (rounded != nullptr && rounded_dtype == KA_BF16)
        hipLaunchKernelGGL(branches_sum_kernel<bf16_t>, dim3(n), dim3(MP_THREADS), 0, stream, x, a, gain_a, ca, b, gain_b, cb, eps, dim,
                           (bf16_t*)rounded);
    else
        hipLaunchKernelGGL(branches_sum_kernel<float>, dim3(n), dim3(MP_THREADS), 0, stream, x, a, gain_a, ca, b, gain_b, cb, eps, dim,
                           (float*)rounded);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// Gated matrix memory: per request and head a state S [d, dv], n [d] and a running maximum m (fp32, in that
// order in `state`, [state rows, heads, d dv + d + 1]), advanced token by token:
//     li = cap tanh(gi / cap),  lf = logsigmoid(cap tanh(gf / cap))          (gi, gf: pre[t, head], pre[t, heads + head])
//     m' = max(lf + m, li);  S' = e^(lf + m - m') S + e^(li - m') k v^T;  n' likewise with k
//     o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6),  q already times q_scale
//     out[t, head dv + j] = o_j / sqrt(mean_j(o^2) + eps) * gain[head dv + j] * sigmoid(gate[t, head dv + j])
// A workgroup per (head, row) walks over the row's tokens (cu_q) in order. The state lives in LDS while it does
// (LDS_STATE) or stays in memory (rows of one token, states too large for LDS). A row without a request
// (row_slot < 0) writes zeros and touches no state.
// ----------------------------------------------------------------------------
struct MemoryArgs {
    const void* q; const void* k; const void* v; const void* gate;     // rows of the activation type, one stride
    long stride;
    const float* pre;              // fp32 [n, 2 heads]
    float* state;
    const int* cu_q;
    const int* row_slot;
    const float* gain;             // fp32 [heads dv] or null
    void* out;
    long out_stride;
    int heads, d, dv, parts;
    float q_scale, cap, eps;
};

template <typename T, bool LDS_STATE>
__global__ void __launch_bounds__(MP_THREADS) matrix_memory_kernel(MemoryArgs a) {
    extern __shared__ float sm[];
    const int head = blockIdx.x, r = blockIdx.y, tid = threadIdx.x;
    const int t0 = a.cu_q[r], t1 = a.cu_q[r + 1];
    if (t0 >= t1) return;
    const int d = a.d, dv = a.dv, parts = a.parts;
    T* out = reinterpret_cast<T*>(a.out);
    const int slot = a.row_slot[r];
    if (slot < 0) {
        for (int t = t0; t < t1; ++t)
            for (int j = tid; j < dv; j += MP_THREADS) out[(size_t)t * a.out_stride + head * dv + j] = ka_from_float<T>(0.f);
        return;
    }
    const int per_head = d * dv + d + 1;
    float* st = a.state + ((size_t)slot * a.heads + head) * per_head;
    float* S = LDS_STATE ? sm : st;
    float* nv = S + d * dv;
    float* qs = sm + (LDS_STATE ? d * dv + d : 0);
    float* ks = qs + d;
    float* vs = ks + d;
    float* part = vs + dv;             // [parts, dv]
    float* red = part + parts * dv;    // [1 + MP_WAVES]
    if (LDS_STATE)
        for (int e = tid; e < d * dv + d; e += MP_THREADS) sm[e] = st[e];
    float m = st[d * dv + d];
    const T* qp = reinterpret_cast<const T*>(a.q);
    const T* kp = reinterpret_cast<const T*>(a.k);
    const T* vp = reinterpret_cast<const T*>(a.v);
    const T* gp = reinterpret_cast<const T*>(a.gate);
    for (int t = t0; t < t1; ++t) {
        const size_t at = (size_t)t * a.stride;
        __syncthreads();               // (the token before is done with qs, ks, vs, part and red)
        for (int e = tid; e < d; e += MP_THREADS) {
            qs[e] = ka_to_float(qp[at + head * d + e]) * a.q_scale;
            ks[e] = ka_to_float(kp[at + head * d + e]);
        }
        for (int j = tid; j < dv; j += MP_THREADS) vs[j] = ka_to_float(vp[at + head * dv + j]);
        const float gi = a.pre[(size_t)t * 2 * a.heads + head], gf = a.pre[(size_t)t * 2 * a.heads + a.heads + head];
        const float li = a.cap * tanhf(gi / a.cap);
        const float z = a.cap * tanhf(gf / a.cap);
        const float lf = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
        const float m_new = fmaxf(lf + m, li);
        const float keep = expf(lf + m - m_new), take = expf(li - m_new);
        m = m_new;
        __syncthreads();
        if (tid < KA_WAVE) {
            float acc = 0.f;
            for (int e = tid; e < d; e += KA_WAVE) {
                const float x = keep * nv[e] + take * ks[e];
                nv[e] = x;
                acc += x * qs[e];
            }
            acc = ka_wave_sum(acc);
            if (tid == 0) red[0] = acc;
        }
        for (int idx = tid; idx < parts * dv; idx += MP_THREADS) {
            const int j = idx % dv, p = idx / dv;
            const float vj = take * vs[j];
            float acc = 0.f;
            // eight numbers of the state in flight at a time (a load behind a store to the same array would wait for it)
            int i = p;
            for (; i + 7 * parts < d; i += 8 * parts) {
                float s8[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) s8[u] = S[(size_t)(i + u * parts) * dv + j];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    s8[u] = keep * s8[u] + ks[i + u * parts] * vj;
                    acc += s8[u] * qs[i + u * parts];
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) S[(size_t)(i + u * parts) * dv + j] = s8[u];
            }
            for (; i < d; i += parts) {
                const float s = keep * S[(size_t)i * dv + j] + ks[i] * vj;
                S[(size_t)i * dv + j] = s;
                acc += s * qs[i];
            }
            part[idx] = acc;
        }
        __syncthreads();
        const float den = fmaxf(fabsf(red[0]), expf(-m_new)) + 1e-6f;
        float o[4];                    // (dv <= 4 * 256)
        float sq = 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = tid + u * MP_THREADS;
            o[u] = 0.f;
            if (j < dv) {
                float acc = 0.f;
                for (int p = 0; p < parts; ++p) acc += part[p * dv + j];
                o[u] = acc / den;
                sq += o[u] * o[u];
            }
        }
        const float rr = 1.0f / sqrtf(mp_block_sum(sq, red + 1) / (float)dv + a.eps);
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int j = tid + u * MP_THREADS;
            if (j < dv) {
                const int c = head * dv + j;
                const float g = gp ? mp_sigmoid(ka_to_float(gp[at + c])) : 1.f;
                out[(size_t)t * a.out_stride + c] = ka_from_float<T>(o[u] * rr * (a.gain ? a.gain[c] : 1.f) * g);
            }
        }
    }
    __syncthreads();
    if (LDS_STATE)
        for (int e = tid; e < d * dv + d; e += MP_THREADS) st[e] = sm[e];
    if (tid == 0) st[d * dv + d] = m;
}

// Floats of LDS that the kernel needs beside the state.
static size_t mm_scratch_floats(int d, int dv, int parts) { return (size_t)2 * d + dv + (size_t)parts * dv + 1 + MP_WAVES; }

constexpr size_t MM_LDS_LIMIT = 128 * 1024;

KA_API int ka_matrix_memory(const void* q, const void* k, const void* v, const void* gate, long stride, int dtype,
                            const float* pre, float* state, int state_rows, const int* cu_q, const int* row_slot,
                            const float* gain, void* out, long out_stride, int n_rows, int heads, int d, int dv,
                            float q_scale, float cap, float eps, int single_tokens, hipStream_t stream) {
    const char* who = "ka_matrix_memory";
    KA_CHECK(n_rows >= 0 && heads > 0 && d > 0 && dv > 0 && state_rows > 0, "%s: bad sizes", who);
    KA_CHECK(dv <= 4 * MP_THREADS, "%s: value size %d above %d", who, dv, 4 * MP_THREADS);
    KA_CHECK(cap > 0.f && eps >= 0.f, "%s: the gates' cap must be positive", who);
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "%s: unsupported dtype %d", who, dtype);
    KA_CHECK(heads <= 65535 && n_rows <= 65535, "%s: too many heads or rows", who);
    if (n_rows == 0) return 0;
    int parts = MP_THREADS / dv;
    parts = parts < 1 ? 1 : (parts > d ? d : parts);
    const size_t scratch = mm_scratch_floats(d, dv, parts) * sizeof(float);
    const size_t with_state = scratch + ((size_t)d * dv + d) * sizeof(float);
    // rows of one token read and write every number of the state once either way: no detour through LDS
    const bool in_lds = !single_tokens && with_state <= MM_LDS_LIMIT;
    KA_CHECK(scratch <= MM_LDS_LIMIT, "%s: heads of %d x %d do not fit", who, d, dv);
    MemoryArgs a{q, k, v, gate, stride, pre, state, cu_q, row_slot, gain, out, out_stride, heads, d, dv, parts, q_scale, cap, eps};
    const dim3 grid(heads, n_rows), block(MP_THREADS);
#define MM_LAUNCH(T, IN_LDS, BYTES)                                                                                        \
    do {                                                                                                                   \
        static bool sized = false;                                                                                         \
        if (!sized) {                                                                                                      \
            (void)hipFuncSetAttribute((const void*)matrix_memory_kernel<T, IN_LDS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)MM_LDS_LIMIT); \
            sized = true;                                                                                                  \
        }                                                                                                                  \
        hipLaunchKernelGGL((matrix_memory_kernel<T, IN_LDS>), grid, block, BYTES, stream, a);                              \
    } while (0)
    if (dtype == KA_F32) {
        if (in_lds) MM_LAUNCH(float, true, with_state);
        else MM_LAUNCH(float, false, scratch);
    } else {
        if (in_lds) MM_LAUNCH(bf16_t, true, with_state);
        else MM_LAUNCH(bf16_t, false, scratch);
    }
#undef MM_LAUNCH
    KA_LAUNCH_CHECK();
    return 0;
}
