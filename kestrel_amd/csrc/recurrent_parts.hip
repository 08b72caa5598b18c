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
// Two launches. The first walks over every row's tokens of this step, whatever they are (a prompt, a portion, one
// token), and leaves the read-outs o in fp32. The columns j of S are independent of each other, so a head is dealt out
// over workgroups by slices of value channels (blockIdx.z) as well as over threads: thread (p, j) of a workgroup keeps
// the NI entries S[p NI .. p NI + NI - 1][j] in registers. Tokens are taken in blocks: r, k, w, v and u r k of a block are
// staged in LDS in fp32 (w computed there; the next block's numbers are already on their way from memory), the threads
// then run the recurrence over the block's tokens with no exchange between them but the LDS reads, leave their partial
// read-outs in LDS, and the partial read-outs of the block are summed a wave per token. Every token's arithmetic is the
// same wherever a step was cut. What a token costs is instructions (a hundred and fifty a wave with a quarter of a head of
// 64 a thread, counted on the GPU), so the fast form (heads that are multiples of 16 channels) gives a thread four key
// channels of one value channel, sixteen value channels a workgroup.
// The second launch normalises, a wave per (token, head). A row without a request (slot < 0) gets zeros.
// The workgroup of head 0, slice 0 also keeps the stream's last row of the portion for the next step's token shift.
// ----------------------------------------------------------------------------
struct DecayArgs {
    const void* r;
    const void* k;
    const void* v;
    long stride;            // of the rows of r, k and v
    const float* pre;       // [n, H d]
    const float* u;         // [H d]
    float* state;           // [slots, state_stride]: S [H, d, d], then the kept row [dim]
    long state_stride;
    const float* x;         // the stream [n, dim] (the kept row comes from it), or null
    int dim;
    const int* cu_q;
    const int* row_slot;
    float* raw;             // [n, H d]: the read-outs before their norm
    int H, d, block_tokens, parts, slice;       // slice: value channels a workgroup
};

constexpr int RP_SLICE = 16;        // value channels a workgroup of the fast form (half as many for heads above 128 channels)

// FAST: d is a multiple of 16; NI = 4 key channels a thread (read from LDS four at a time), RP_SLICE value channels a
// workgroup. Otherwise any d, the whole head a workgroup.
template <typename T, int NI, bool FAST>
__global__ void __launch_bounds__(!FAST && NI == 64 ? 1024 : 512) decayed_memory_kernel(DecayArgs a) {
    extern __shared__ float sm[];
    const int head = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
    const int d = a.d, TB = a.block_tokens, P = a.parts, dj = a.slice;
    const int j0 = blockIdx.z * dj;
    const int t0 = a.cu_q[row], t1 = a.cu_q[row + 1];
    if (t0 >= t1) return;
    const int slot = a.row_slot[row];
    const int wave = tid / KA_WAVE, lane = tid % KA_WAVE, n_waves = blockDim.x / KA_WAVE;
    if (slot < 0) {
        for (int e = tid; e < (t1 - t0) * dj; e += blockDim.x)
            a.raw[(size_t)(t0 + e / dj) * a.H * d + (size_t)head * d + j0 + e % dj] = 0.f;
        return;
    }
    float* rs = sm;                         // [TB][d]
    float* ks = rs + (size_t)TB * d;
    float* ws = ks + (size_t)TB * d;
    float* bs = ws + (size_t)TB * d;        // [TB][d]: r_i u_i k_i, whose sum over i is the bonus term's factor
    float* vs = bs + (size_t)TB * d;        // [TB][dj]
    float* po = vs + (size_t)TB * dj;       // [TB][P][dj]
    const int jl = tid % dj, p = tid / dj;
    const int j = j0 + jl;
    const bool works = p < P;
    const int i0 = p * NI;
    float* S_mem = a.state + (size_t)slot * a.state_stride + (size_t)head * d * d;
    float S[NI];
#pragma unroll
    for (int ii = 0; ii < NI; ++ii) S[ii] = works && i0 + ii < d ? S_mem[(size_t)(i0 + ii) * d + j] : 0.f;
    const T* rp = reinterpret_cast<const T*>(a.r) + (size_t)head * d;
    const T* kp = reinterpret_cast<const T*>(a.k) + (size_t)head * d;
    const T* vp = reinterpret_cast<const T*>(a.v) + (size_t)head * d;
    const float* up = a.u + (size_t)head * d;
    // what a thread fetches of a block: its elements e = tid + m * threads of r, k, the decay's pre-activation and (of the
    // slice's channels) v. The next block's are asked for before the current block is computed.
    constexpr int RP_FETCH = FAST ? 4 : (NI == 64 ? 2 : 8);      // (the host sizes the block so that a thread has at most this many)
    T fr[RP_FETCH], fk[RP_FETCH], fv[RP_FETCH];
    float fw[RP_FETCH];
    // (which token of a block and which channel an element is does not change from block to block: the divisions are done once)
    int e_tok[RP_FETCH], e_ch[RP_FETCH], v_tok[RP_FETCH], v_ch[RP_FETCH];
    float e_u[RP_FETCH];
#pragma unroll
    for (int m = 0; m < RP_FETCH; ++m) {
        const int e = tid + m * (int)blockDim.x;
        e_tok[m] = e / d;
        e_ch[m] = e % d;
        v_tok[m] = e / dj;
        v_ch[m] = e % dj;
        e_u[m] = up[e_ch[m]];
    }
    auto fetch = [&](int tb) {
        const int nb = min(TB, t1 - tb);
#pragma unroll
        for (int m = 0; m < RP_FETCH; ++m) {
            if (e_tok[m] < nb) {
                const size_t at = (size_t)(tb + e_tok[m]) * a.stride + e_ch[m];
                fr[m] = rp[at];
                fk[m] = kp[at];
                fw[m] = a.pre[(size_t)(tb + e_tok[m]) * a.H * d + (size_t)head * d + e_ch[m]];
            }
            if (v_tok[m] < nb) fv[m] = vp[(size_t)(tb + v_tok[m]) * a.stride + j0 + v_ch[m]];
        }
    };
    // This wave's LDS writes done, then everybody's: what __syncthreads() does too, but that one also waits for every load
    // and store in flight, which is the next block's numbers on their way from memory and the read-outs on their way there.
    auto lds_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(0xc07f);      // lgkmcnt(0), the other counters at their maximum
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    fetch(t0);
    for (int tb = t0; tb < t1; tb += TB) {
        const int nb = min(TB, t1 - tb);
#pragma unroll
        for (int m = 0; m < RP_FETCH; ++m) {
            const int e = tid + m * (int)blockDim.x;
            if (e_tok[m] < nb) {
                const float r = ka_to_float(fr[m]), k = ka_to_float(fk[m]);
                rs[e] = r;
                ks[e] = k;
                // (bf16 runs take the hardware's exponential: its error is far below what the projections' rounding leaves)
                ws[e] = sizeof(T) == 2 ? __expf(-__expf(fw[m])) : expf(-expf(fw[m]));
                bs[e] = r * e_u[m] * k;
            }
            if (v_tok[m] < nb) vs[e] = ka_to_float(fv[m]);
        }
        if (tb + TB < t1) fetch(tb + TB);
        lds_barrier();
        if constexpr (FAST) {
            static_assert(!FAST || NI == 4, "the fast form reads four key channels at a time");
            // A wave has its SIMD to itself, so nothing but its own next loads can hide a load's way through LDS: the
            // block's tokens are unrolled, token tt + 1's numbers are asked for before token tt's sums, and the partial
            // read-outs stay in registers until the block is done (a store between the loads would keep them in order).
            constexpr int RP_BLOCK = 16;                 // (the host gives a block at most this many tokens)
            if (works) {
                float outs[RP_BLOCK];
                // (four tokens ahead: a trip through LDS, with the workgroup's other waves asking too, takes as long as three
                // or four tokens' sums)
                constexpr int RP_AHEAD = 4;
                float4 rq[RP_AHEAD], kq[RP_AHEAD], wq[RP_AHEAD];
                float vq[RP_AHEAD];
#pragma unroll
                for (int q = 0; q < RP_AHEAD; ++q) {
                    if (q < nb) {
                        rq[q] = *reinterpret_cast<const float4*>(rs + q * d + i0);
                        kq[q] = *reinterpret_cast<const float4*>(ks + q * d + i0);
                        wq[q] = *reinterpret_cast<const float4*>(ws + q * d + i0);
                        vq[q] = vs[q * dj + jl];
                    }
                }
#pragma unroll
                for (int tt = 0; tt < RP_BLOCK; ++tt) {
                    if (tt < nb) {
                        const float4 r4 = rq[tt % RP_AHEAD], k4 = kq[tt % RP_AHEAD], w4 = wq[tt % RP_AHEAD];
                        const float vj = vq[tt % RP_AHEAD];
                        if (tt + RP_AHEAD < nb) {
                            rq[tt % RP_AHEAD] = *reinterpret_cast<const float4*>(rs + (tt + RP_AHEAD) * d + i0);
                            kq[tt % RP_AHEAD] = *reinterpret_cast<const float4*>(ks + (tt + RP_AHEAD) * d + i0);
                            wq[tt % RP_AHEAD] = *reinterpret_cast<const float4*>(ws + (tt + RP_AHEAD) * d + i0);
                            vq[tt % RP_AHEAD] = vs[(tt + RP_AHEAD) * dj + jl];
                        }
                        float acc = r4.x * S[0];
                        S[0] = fmaf(w4.x, S[0], k4.x * vj);
                        acc = fmaf(r4.y, S[1], acc);
                        S[1] = fmaf(w4.y, S[1], k4.y * vj);
                        acc = fmaf(r4.z, S[2], acc);
                        S[2] = fmaf(w4.z, S[2], k4.z * vj);
                        acc = fmaf(r4.w, S[3], acc);
                        S[3] = fmaf(w4.w, S[3], k4.w * vj);
                        outs[tt] = acc;
                    }
                }
                // With 16 value channels a workgroup a wave holds four parts of every channel, 16 lanes apart: they meet
                // inside the wave (two swaps of rows and halves), and one lane in four writes.
                const bool meet = dj == 16;
#pragma unroll
                for (int tt = 0; tt < RP_BLOCK; ++tt) {
                    if (tt < nb) {
                        float y = outs[tt];
                        if (meet) {
                            float y1, y2;
                            ka_lanes_pair<16>(y, y1, y2);
                            y = y1 + y2;
                            ka_lanes_pair<32>(y, y1, y2);
                            y = y1 + y2;
                            if (lane < 16) po[((size_t)tt * P + wave * 4) * dj + jl] = y;
                        } else {
                            po[((size_t)tt * P + p) * dj + jl] = y;
                        }
                    }
                }
            }
        } else if (works) {
            for (int tt = 0; tt < nb; ++tt) {
                const float vj = vs[tt * dj + jl];
                const float* r_t = rs + tt * d + i0;
                const float* k_t = ks + tt * d + i0;
                const float* w_t = ws + tt * d + i0;
                float acc = 0.f;
#pragma unroll
                for (int ii = 0; ii < NI; ++ii) {
                    if (i0 + ii < d) {
                        acc = fmaf(r_t[ii], S[ii], acc);
                        S[ii] = fmaf(w_t[ii], S[ii], k_t[ii] * vj);
                    }
                }
                po[((size_t)tt * P + p) * dj + jl] = acc;
            }
        }
        lds_barrier();
        // read-outs of the block: a wave per token; the bonus term's factor is a sum over all key channels, the partial
        // read-outs are summed per value channel of the slice
        if (FAST && dj == 16 && (int)blockDim.x >= TB * 16) {
            // an output a thread: token tid / 16, channel tid % 16; the 16 lanes of a token sum u r k over the key channels
            // between them (a row of the vector unit's lane moves)
            const int tt = tid / 16, c = tid % 16;
            float part = 0.f;
            if (tt < nb)
                for (int q = c; q < d; q += 16) part += bs[tt * d + q];
            const float bonus = ka_lanes_reduce<1, 16>(part, KaSum{});
            if (tt < nb) {
                float y = bonus * vs[tt * dj + c];
                for (int pp = 0; pp < P; pp += 4) y += po[((size_t)tt * P + pp) * dj + c];
                a.raw[(size_t)(tb + tt) * a.H * d + (size_t)head * d + j0 + c] = y;
            }
        } else
        for (int tt = wave; tt < nb; tt += n_waves) {
            float bonus = 0.f;
            for (int c = lane; c < d; c += KA_WAVE) bonus += bs[tt * d + c];
            bonus = ka_wave_sum(bonus);
            for (int c = lane; c < dj; c += KA_WAVE) {
                float y = bonus * vs[tt * dj + c];
                // (the fast form with 16 channels a workgroup has left one sum a wave, at the place of the wave's first part)
                const int hop = FAST && dj == 16 ? 4 : 1;
                for (int pp = 0; pp < P; pp += hop) y += po[((size_t)tt * P + pp) * dj + c];
                a.raw[(size_t)(tb + tt) * a.H * d + (size_t)head * d + j0 + c] = y;
            }
        }
        lds_barrier();
    }
    if (works) {
#pragma unroll
        for (int ii = 0; ii < NI; ++ii)
            if (i0 + ii < d) S_mem[(size_t)(i0 + ii) * d + j] = S[ii];
    }
    if (head == 0 && blockIdx.z == 0 && a.x != nullptr) {
        float* kept = a.state + (size_t)slot * a.state_stride + (size_t)a.H * d * d;
        const float* last = a.x + (size_t)(t1 - 1) * a.dim;
        for (int c = tid; c < a.dim; c += blockDim.x) kept[c] = last[c];
    }
}

// out[t, h, :] = raw[t, h, :] / sqrt(mean(raw[t, h, :]^2) + eps) * gain[h, :] * gate[t, h, :]: a wave per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
decayed_readout_kernel(const float* __restrict__ raw, const float* __restrict__ gain, const T* __restrict__ gate, long gate_stride,
                       T* __restrict__ out, long out_stride, int n, int H, int d, float eps) {
    const int pair = blockIdx.x * (blockDim.x / KA_WAVE) + threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    if (pair >= n * H) return;
    const int t = pair / H, head = pair % H;
    const float* o = raw + (size_t)t * H * d + (size_t)head * d;
    float ss = 0.f;
    for (int c = lane; c < d; c += KA_WAVE) ss = fmaf(o[c], o[c], ss);
    const float inv = 1.0f / sqrtf(ka_wave_sum(ss) / (float)d + eps);
    for (int c = lane; c < d; c += KA_WAVE)
        out[(size_t)t * out_stride + (size_t)head * d + c] =
            ka_from_float<T>(o[c] * inv * gain[(size_t)head * d + c] * ka_to_float(gate[(size_t)t * gate_stride + (size_t)head * d + c]));
}

// How the general form cuts a head of d channels: NI state entries a thread, `parts` threads a value channel.
static bool decay_shape(int d, int* ni, int* parts) {
    if (d <= 0 || d > 256) return false;
    for (int cand : {16, 32, 64}) {
        const int pp = (d + cand - 1) / cand;
        if ((long)pp * d <= (cand == 64 ? 1024 : 512)) {
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

// raw: fp32 scratch [n, H d] of the caller's.
KA_API int ka_decayed_memory(const void* r, const void* k, const void* v, const void* gate, long stride, int dtype, const float* pre,
                             const float* u, const float* gain, float* state, long state_stride, const float* x, int dim,
                             const int* cu_q, const int* row_slot, void* out, long out_stride, int n, int n_rows, int H, int d, float eps,
                             float* raw, hipStream_t stream) {
    const char* who = "ka_decayed_memory";
    KA_CHECK(n >= 0 && n_rows >= 0 && H > 0 && d > 0 && eps >= 0.f && raw != nullptr, "%s: bad sizes", who);
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "%s: unsupported dtype %d", who, dtype);
    int ni = 0, parts = 0;
    KA_CHECK(decay_shape(d, &ni, &parts), "%s: heads of %d channels are not covered (up to 256)", who, d);
    KA_CHECK(state_stride >= (long)H * d * d + (x ? dim : 0), "%s: the state rows are too short", who);
    KA_CHECK(H <= 65535 && n_rows <= 65535, "%s: too many heads or rows", who);
    if (n_rows == 0 || n == 0) return 0;
    const bool fast = d % RP_SLICE == 0;
    int slice = d, fetch = ni == 64 ? 2 : 8;
    if (fast) {
        ni = 4;
        parts = d / 4;
        slice = d > 128 ? RP_SLICE / 2 : RP_SLICE;          // (at most 512 threads a workgroup)
        fetch = 4;
    }
    const int threads = ((parts * slice + KA_WAVE - 1) / KA_WAVE) * KA_WAVE;
    int block_tokens = 49152 / (4 * (4 * d + slice * (1 + parts)));
    block_tokens = block_tokens < 1 ? 1 : (block_tokens > 16 ? 16 : block_tokens);
    if (block_tokens > fetch * threads / d) block_tokens = fetch * threads / d;          // (what a thread fetches of a block)
    if (block_tokens < 1) block_tokens = 1;
    const size_t lds = (size_t)block_tokens * (4 * d + slice * (1 + parts)) * sizeof(float);
    DecayArgs a{r, k, v, stride, pre, u, state, state_stride, x, dim, cu_q, row_slot, raw, H, d, block_tokens, parts, slice};
    dim3 grid(H, n_rows, d / slice);
#define RP_LAUNCH(T, NI, FAST) hipLaunchKernelGGL((decayed_memory_kernel<T, NI, FAST>), grid, dim3(threads), lds, stream, a)
#define RP_LAUNCH_ALL(T)                                                            \
    if (fast) RP_LAUNCH(T, 4, true);                                                \
    else if (ni == 16) RP_LAUNCH(T, 16, false);                                     \
    else if (ni == 32) RP_LAUNCH(T, 32, false);                                     \
    else RP_LAUNCH(T, 64, false);
    if (dtype == KA_F32) { RP_LAUNCH_ALL(float) } else { RP_LAUNCH_ALL(bf16_t) }
#undef RP_LAUNCH_ALL
#undef RP_LAUNCH
    KA_LAUNCH_CHECK();
    const int pairs = n * H;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(decayed_readout_kernel<float>, dim3((pairs + 3) / 4), dim3(256), 0, stream, raw, gain, (const float*)gate, stride,
                           (float*)out, out_stride, n, H, d, eps);
    else
        hipLaunchKernelGGL(decayed_readout_kernel<bf16_t>, dim3((pairs + 3) / 4), dim3(256), 0, stream, raw, gain, (const bf16_t*)gate, stride,
                           (bf16_t*)out, out_stride, n, H, d, eps);
    KA_LAUNCH_CHECK();
    return 0;
}
