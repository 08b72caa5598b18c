// Kernels of a recurrent mixer whose state decays channel by channel (time mixing in the manner of RWKV): the token
// shift that feeds its projections, and the recurrence itself. fp32 or bf16 storage of what the projections made; the
// shift, the decay, the state, the read-out and its norm are fp32.
#include "ka_common.h"

constexpr int RP_THREADS = 256;

// ----------------------------------------------------------------------------
// Token shift: for every token t of the packed step and each of `n_mixes` learned vectors mu_s,
//     out[s][t] = x[t] + (x'[t] - x[t]) * mu_s
// with x'[t] the stream's row of the token before t in its sequence: row t - 1 of the step, or, for the first token of a
// request's portion, the row kept in the request's state (zeros for a new request). A row without a request
// (slot < 0) has zeros before its first token. x fp32 [n, dim]; out [n_mixes][n][dim] of type T.
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(RP_THREADS)
token_shift_kernel(const float* __restrict__ x, const float* __restrict__ kept, long kept_stride, const float* __restrict__ mu,
                   const int* __restrict__ token_row, const int* __restrict__ cu_q, const int* __restrict__ row_slot,
                   T* __restrict__ out, int n, int dim, int n_mixes) {
    const int t = blockIdx.x;
    const int row = token_row[t];
    const bool first = t == cu_q[row];
    const int slot = row_slot[row];
    const float* before = first ? (slot >= 0 ? kept + (size_t)slot * kept_stride : nullptr) : x + (size_t)(t - 1) * dim;
    const float* here = x + (size_t)t * dim;
    for (int c = threadIdx.x; c < dim; c += RP_THREADS) {
        const float h = here[c];
        const float d = (before ? before[c] : 0.f) - h;
        for (int s = 0; s < n_mixes; ++s)
            out[((size_t)s * n + t) * dim + c] = ka_from_float<T>(fmaf(d, mu[(size_t)s * dim + c], h));
    }
}

KA_API int ka_token_shift(const float* x, const float* kept, long kept_stride, const float* mu, const int* token_row,
                          const int* cu_q, const int* row_slot, void* out, int out_dtype, int n, int dim, int n_mixes,
                          hipStream_t stream) {
    KA_CHECK(n >= 0 && dim > 0 && n_mixes > 0 && kept_stride >= dim, "ka_token_shift: bad sizes n=%d dim=%d mixes=%d", n, dim, n_mixes);
    KA_CHECK(out_dtype == KA_F32 || out_dtype == KA_BF16, "ka_token_shift: unsupported dtype %d", out_dtype);
    if (n == 0) return 0;
    if (out_dtype == KA_F32)
        hipLaunchKernelGGL(token_shift_kernel<float>, dim3(n), dim3(RP_THREADS), 0, stream, x, kept, kept_stride, mu, token_row, cu_q,
                           row_slot, (float*)out, n, dim, n_mixes);
    else
        hipLaunchKernelGGL(token_shift_kernel<bf16_t>, dim3(n), dim3(RP_THREADS), 0, stream, x, kept, kept_stride, mu, token_row, cu_q,
                           row_slot, (bf16_t*)out, n, dim, n_mixes);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The recurrence. Per head a state S [d, d] (key channel i, value channel j), fp32, kept per request. For every token
// of a row, in order, with w_i = exp(-exp(pre_i)) the decay of key channel i:
//     o_j = sum_i r_i (S_ij + u_i k_i v_j)        (the bonus u counts for the token's own key only)
//     S_ij <- w_i S_ij + k_i v_j
// then o is divided by its root mean square over the head (eps), multiplied by gain and by the gate.
//
// A workgroup owns one head of one row and walks over the row's tokens of this step, whatever they are (a prompt, a
// portion, one token). Thread (p, j) keeps the NI entries S[p NI .. p NI + NI - 1][j] in registers. Tokens are taken
// in blocks: r, k, w and v of a block are staged in LDS in fp32 (w computed there), the threads then run the
// recurrence over the block's tokens with no exchange between them but the LDS reads, leave their partial read-outs
// in LDS, and the read-outs of the block are summed, normalised, gated and stored a wave per token. Every token's
// arithmetic is the same wherever a step was cut. A row without a request (slot < 0) writes zeros.
// The workgroup of head 0 also keeps the stream's last row of the portion for the next step's token shift.
// ----------------------------------------------------------------------------
struct DecayArgs {
    const void* r;
    const void* k;
    const void* v;
    const void* gate;
    long stride;            // of the rows of r, k, v and gate
    const float* pre;       // [n, H d]
    const float* u;         // [H d]
    const float* gain;      // [H d]
    float* state;           // [slots, state_stride]: S [H, d, d], then the kept row [dim]
    long state_stride;
    const float* x;         // the stream [n, dim] (the kept row comes from it), or null
    int dim;
    const int* cu_q;
    const int* row_slot;
    void* out;
    long out_stride;
    int H, d, block_tokens, parts;
    float eps;
};

// FULL: d is a multiple of NI (no thread's range of key channels ends early) and of 4 (the LDS rows are read four at a time).
template <typename T, int NI, bool FULL>
__global__ void __launch_bounds__(1024) decayed_memory_kernel(DecayArgs a) {
    extern __shared__ float sm[];
    const int head = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
    const int d = a.d, TB = a.block_tokens, P = a.parts;
    const int t0 = a.cu_q[row], t1 = a.cu_q[row + 1];
    if (t0 >= t1) return;
    const int slot = a.row_slot[row];
    const int wave = tid / KA_WAVE, lane = tid % KA_WAVE, n_waves = blockDim.x / KA_WAVE;
    T* out = reinterpret_cast<T*>(a.out);
    if (slot < 0) {
        for (int e = tid; e < (t1 - t0) * d; e += blockDim.x)
            out[(size_t)(t0 + e / d) * a.out_stride + (size_t)head * d + e % d] = ka_from_float<T>(0.f);
        return;
    }
    float* rs = sm;                         // [TB][d]
    float* ks = rs + (size_t)TB * d;
    float* ws = ks + (size_t)TB * d;
    float* vs = ws + (size_t)TB * d;
    float* bs = vs + (size_t)TB * d;        // [TB][d]: r_i u_i k_i, whose sum over i is the bonus term's factor
    float* po = bs + (size_t)TB * d;        // [TB][P][d]
    const int j = tid % d, p = tid / d;
    const bool works = p < P;
    const int i0 = p * NI;
    float* S_mem = a.state + (size_t)slot * a.state_stride + (size_t)head * d * d;
    float S[NI];
#pragma unroll
    for (int ii = 0; ii < NI; ++ii) S[ii] = works && i0 + ii < d ? S_mem[(size_t)(i0 + ii) * d + j] : 0.f;
    const T* rp = reinterpret_cast<const T*>(a.r) + (size_t)head * d;
    const T* kp = reinterpret_cast<const T*>(a.k) + (size_t)head * d;
    const T* vp = reinterpret_cast<const T*>(a.v) + (size_t)head * d;
    const T* gp = reinterpret_cast<const T*>(a.gate) + (size_t)head * d;
    const float* up = a.u + (size_t)head * d;
    const float* gain = a.gain + (size_t)head * d;
    for (int tb = t0; tb < t1; tb += TB) {
        const int nb = min(TB, t1 - tb);
        for (int e = tid; e < nb * d; e += blockDim.x) {
            const int tt = e / d, c = e % d;
            const size_t at = (size_t)(tb + tt) * a.stride + c;
            rs[e] = ka_to_float(rp[at]);
            ks[e] = ka_to_float(kp[at]);
            vs[e] = ka_to_float(vp[at]);
            ws[e] = expf(-expf(a.pre[(size_t)(tb + tt) * a.H * d + (size_t)head * d + c]));
            bs[e] = rs[e] * up[c] * ks[e];
        }
        __syncthreads();
        if (works) {
            for (int tt = 0; tt < nb; ++tt) {
                const float vj = vs[tt * d + j];
                const float* r_t = rs + tt * d + i0;
                const float* k_t = ks + tt * d + i0;
                const float* w_t = ws + tt * d + i0;
                float acc = 0.f;
                if constexpr (FULL) {
#pragma unroll
                    for (int ii = 0; ii < NI; ii += 4) {
                        const float4 r4 = *reinterpret_cast<const float4*>(r_t + ii);
                        const float4 k4 = *reinterpret_cast<const float4*>(k_t + ii);
                        const float4 w4 = *reinterpret_cast<const float4*>(w_t + ii);
                        acc = fmaf(r4.x, S[ii], acc);
                        S[ii] = fmaf(w4.x, S[ii], k4.x * vj);
                        acc = fmaf(r4.y, S[ii + 1], acc);
                        S[ii + 1] = fmaf(w4.y, S[ii + 1], k4.y * vj);
                        acc = fmaf(r4.z, S[ii + 2], acc);
                        S[ii + 2] = fmaf(w4.z, S[ii + 2], k4.z * vj);
                        acc = fmaf(r4.w, S[ii + 3], acc);
                        S[ii + 3] = fmaf(w4.w, S[ii + 3], k4.w * vj);
                    }
                } else {
#pragma unroll
                    for (int ii = 0; ii < NI; ++ii) {
                        if (i0 + ii < d) {
                            acc = fmaf(r_t[ii], S[ii], acc);
                            S[ii] = fmaf(w_t[ii], S[ii], k_t[ii] * vj);
                        }
                    }
                }
                po[((size_t)tt * P + p) * d + j] = acc;
            }
        }
        __syncthreads();
        // read-outs of the block: a wave per token, lanes over the value channels
        for (int tt = wave; tt < nb; tt += n_waves) {
            float o[4];
            float ss = 0.f, bonus = 0.f;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if (lane + q * KA_WAVE < d) bonus += bs[tt * d + lane + q * KA_WAVE];
            bonus = ka_wave_sum(bonus);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = lane + q * KA_WAVE;
                o[q] = 0.f;
                if (c < d) {
                    float y = bonus * vs[tt * d + c];
                    for (int pp = 0; pp < P; ++pp) y += po[((size_t)tt * P + pp) * d + c];
                    o[q] = y;
                    ss = fmaf(y, y, ss);
                }
            }
            const float inv = 1.0f / sqrtf(ka_wave_sum(ss) / (float)d + a.eps);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = lane + q * KA_WAVE;
                if (c < d) {
                    const size_t at = (size_t)(tb + tt);
                    const float g = ka_to_float(gp[at * a.stride + c]);
                    out[at * a.out_stride + (size_t)head * d + c] = ka_from_float<T>(o[q] * inv * gain[c] * g);
                }
            }
        }
        __syncthreads();
    }
    if (works) {
#pragma unroll
        for (int ii = 0; ii < NI; ++ii)
            if (i0 + ii < d) S_mem[(size_t)(i0 + ii) * d + j] = S[ii];
    }
    if (head == 0 && a.x != nullptr) {
        float* kept = a.state + (size_t)slot * a.state_stride + (size_t)a.H * d * d;
        const float* last = a.x + (size_t)(t1 - 1) * a.dim;
        for (int c = tid; c < a.dim; c += blockDim.x) kept[c] = last[c];
    }
}

// How the kernel cuts a head of d channels: NI state entries a thread, `parts` threads a value channel.
static bool decay_shape(int d, int* ni, int* parts) {
    if (d <= 0 || d > 256) return false;
    for (int cand : {4, 8, 16, 32, 64}) {
        const int pp = (d + cand - 1) / cand;
        if ((long)pp * d <= 1024) {
            *ni = cand;
            *parts = pp;
            return true;
        }
    }
    return false;
}

KA_API int ka_decayed_memory_supported(int d) {
    int ni, parts;
    return decay_shape(d, &ni, &parts) ? 1 : 0;
}

KA_API int ka_decayed_memory(const void* r, const void* k, const void* v, const void* gate, long stride, int dtype, const float* pre,
                             const float* u, const float* gain, float* state, long state_stride, const float* x, int dim,
                             const int* cu_q, const int* row_slot, void* out, long out_stride, int n_rows, int H, int d, float eps,
                             hipStream_t stream) {
    const char* who = "ka_decayed_memory";
    KA_CHECK(n_rows >= 0 && H > 0 && d > 0 && eps >= 0.f, "%s: bad sizes", who);
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "%s: unsupported dtype %d", who, dtype);
    int ni = 0, parts = 0;
    KA_CHECK(decay_shape(d, &ni, &parts), "%s: heads of %d channels are not covered (up to 256)", who, d);
    KA_CHECK(state_stride >= (long)H * d * d + (x ? dim : 0), "%s: the state rows are too short", who);
    KA_CHECK(H <= 65535 && n_rows <= 65535, "%s: too many heads or rows", who);
    if (n_rows == 0) return 0;
    int block_tokens = 49152 / (d * 4 * (5 + parts));
    block_tokens = block_tokens < 1 ? 1 : (block_tokens > 16 ? 16 : block_tokens);
    const int threads = ((parts * d + KA_WAVE - 1) / KA_WAVE) * KA_WAVE;
    const size_t lds = (size_t)block_tokens * d * (5 + parts) * sizeof(float);
    const bool full = d % ni == 0 && d % 4 == 0;
    DecayArgs a{r, k, v, gate, stride, pre, u, gain, state, state_stride, x, dim, cu_q, row_slot, out, out_stride, H, d, block_tokens, parts, eps};
    dim3 grid(H, n_rows);
#define RP_LAUNCH(T, NI)                                                                                             \
    if (ni == NI) {                                                                                                  \
        if (full) hipLaunchKernelGGL((decayed_memory_kernel<T, NI, true>), grid, dim3(threads), lds, stream, a);     \
        else hipLaunchKernelGGL((decayed_memory_kernel<T, NI, false>), grid, dim3(threads), lds, stream, a);         \
    }
#define RP_LAUNCH_ALL(T) RP_LAUNCH(T, 4) RP_LAUNCH(T, 8) RP_LAUNCH(T, 16) RP_LAUNCH(T, 32) RP_LAUNCH(T, 64)
    if (dtype == KA_F32) { RP_LAUNCH_ALL(float) } else { RP_LAUNCH_ALL(bf16_t) }
#undef RP_LAUNCH_ALL
#undef RP_LAUNCH
    KA_LAUNCH_CHECK();
    return 0;
}
