// Kernels of a routed mixture of gated feed-forwards: the router's choice, the experts' linears for every (token,
// choice) pair by itself (any sizes, fp32 or bf16 storage, fp32 sums in a fixed order), the list of pairs by expert
// that the matrix-core kernel of the bf16 path walks over, and the weighted sum of what the experts returned.
//
// A pair is p = token * top + choice. chosen[p] names the router's output that the token chose there: a number below
// n_experts is an expert with weights, a number from n_experts on an identity expert whose output is the token's input.
#include "ka_common.h"

constexpr int EX_MAX_OUTPUTS = 512;             // router outputs a wave can hold (8 a lane)
constexpr int EX_PER_LANE = EX_MAX_OUTPUTS / KA_WAVE;
constexpr int EX_MAX_GROUPS = 64;

// The largest value of a wave and the lowest index that holds it, in every lane.
__device__ __forceinline__ void ex_wave_argmax(float& v, int& i) {
#pragma unroll
    for (int step = 1; step < KA_WAVE; step <<= 1) {
        const float ov = __shfl_xor(v, step);
        const int oi = __shfl_xor(i, step);
        if (ov > v || (ov == v && oi < i)) {
            v = ov;
            i = oi;
        }
    }
}

// ----------------------------------------------------------------------------
// The router's choice, a wave per token. logits fp32 [n, >= R] (rows `stride` apart), R router outputs.
//     s = softmax(logits);  choice = s + correction (correction optional)
//     n_groups > 0: the outputs form n_groups equal groups of neighbours, a group's score is its largest choice score,
//       and only outputs of the `keep` best groups can be chosen;
//     the `top` outputs with the largest choice scores are chosen (the lower index wins a tie);
//     weights: their s divided by the sum of the chosen s (+ 1e-20), times scale.
// chosen int32 [n, top], weights fp32 [n, top].
// ----------------------------------------------------------------------------
__global__ void __launch_bounds__(KA_WAVE)
route_kernel(const float* __restrict__ logits, long stride, const float* __restrict__ correction, int R, int top, int n_groups,
             int keep, float scale, int* __restrict__ chosen, float* __restrict__ weights) {
    __shared__ float choice_s[EX_MAX_OUTPUTS];
    __shared__ float group_s[EX_MAX_GROUPS];
    __shared__ int allowed_s[EX_MAX_GROUPS];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * stride;
    float s[EX_PER_LANE], c[EX_PER_LANE];
    float top_z = -INFINITY;
#pragma unroll
    for (int q = 0; q < EX_PER_LANE; ++q) {
        const int r = lane + q * KA_WAVE;
        s[q] = r < R ? z[r] : -INFINITY;
        top_z = fmaxf(top_z, s[q]);
    }
    top_z = ka_wave_max(top_z);
    float total = 0.f;
#pragma unroll
    for (int q = 0; q < EX_PER_LANE; ++q) {
        s[q] = lane + q * KA_WAVE < R ? expf(s[q] - top_z) : 0.f;
        total += s[q];
    }
    total = ka_wave_sum(total);
#pragma unroll
    for (int q = 0; q < EX_PER_LANE; ++q) {
        const int r = lane + q * KA_WAVE;
        s[q] = s[q] / total;
        c[q] = r < R ? s[q] + (correction ? correction[r] : 0.f) : -INFINITY;
        if (r < R) choice_s[r] = c[q];
    }
    if (n_groups > 0) {
        const int per = R / n_groups;
        __syncthreads();
        if (lane < n_groups) {
            float best = -INFINITY;
            for (int m = 0; m < per; ++m) best = fmaxf(best, choice_s[lane * per + m]);
            group_s[lane] = best;
            allowed_s[lane] = 0;
        }
        __syncthreads();
        for (int turn = 0; turn < keep; ++turn) {
            float v = lane < n_groups && !allowed_s[lane] ? group_s[lane] : -INFINITY;
            int i = lane < n_groups && !allowed_s[lane] ? lane : 0x7fffffff;
            ex_wave_argmax(v, i);
            __syncthreads();
            if (lane == 0 && i < n_groups) allowed_s[i] = 1;
            __syncthreads();
        }
#pragma unroll
        for (int q = 0; q < EX_PER_LANE; ++q) {
            const int r = lane + q * KA_WAVE;
            if (r < R && !allowed_s[r / per]) c[q] = -INFINITY;
        }
    }
    float sum = 0.f;
    float mine_w = 0.f;          // lane k keeps the k-th chosen score
    int mine_i = 0;
    unsigned taken = 0;          // bit q: this lane's entry q is chosen already
    for (int k = 0; k < top; ++k) {
        float v = -INFINITY;
        int i = 0x7fffffff;
#pragma unroll
        for (int q = 0; q < EX_PER_LANE; ++q) {
            const int r = lane + q * KA_WAVE;
            if (r < R && !(taken >> q & 1) && (c[q] > v || i == 0x7fffffff)) {
                v = c[q];
                i = r;
            }
        }
        ex_wave_argmax(v, i);
        float sv = 0.f;
#pragma unroll
        for (int q = 0; q < EX_PER_LANE; ++q)
            if (lane + q * KA_WAVE == i) {
                taken |= 1u << q;
                sv = s[q];
            }
        sv = ka_wave_sum(sv);    // (one lane holds it, the others 0)
        sum += sv;
        if (lane == k % KA_WAVE) {
            // (more than a wave of choices would need more than one register a lane: the entry point refuses it)
            mine_w = sv;
            mine_i = i;
        }
    }
    if (lane < top) {
        chosen[(size_t)t * top + lane] = mine_i;
        weights[(size_t)t * top + lane] = mine_w / (sum + 1e-20f) * scale;
    }
}

KA_API int ka_route(const float* logits, long stride, const float* correction, int n, int R, int top, int n_groups, int keep,
                    float scale, int* chosen, float* weights, hipStream_t stream) {
    const char* who = "ka_route";
    KA_CHECK(n >= 0 && R > 0 && R <= EX_MAX_OUTPUTS && stride >= R, "%s: %d router outputs (at most %d)", who, R, EX_MAX_OUTPUTS);
    KA_CHECK(top > 0 && top <= R && top <= KA_WAVE, "%s: %d choices of %d", who, top, R);
    KA_CHECK(n_groups >= 0 && n_groups <= EX_MAX_GROUPS && (n_groups == 0 || (R % n_groups == 0 && keep > 0 && keep <= n_groups)),
             "%s: %d groups of which %d are kept do not divide %d outputs", who, n_groups, keep, R);
    KA_CHECK(n_groups == 0 || keep * (R / n_groups) >= top, "%s: %d kept groups hold fewer than %d outputs", who, keep, top);
    if (n == 0) return 0;
    hipLaunchKernelGGL(route_kernel, dim3(n), dim3(KA_WAVE), 0, stream, logits, stride, correction, R, top, n_groups, keep, scale,
                       chosen, weights);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The linear of every pair's expert, pair by pair: out[p] = act(a[p / a_div] W_e^T) with e = chosen[p] and W [E, N, K].
// Gated (KA_ACT_GATED): rows 2j and 2j + 1 of W_e are gate and value of output j. A pair whose choice is no expert with
// weights (>= E) is passed over. A workgroup takes EX_COLS outputs of one pair; the input row lies in LDS as fp32; a wave
// computes an output as lanes' partial sums over K met in a fixed tree.
// ----------------------------------------------------------------------------
constexpr int EX_COLS = 16;

template <typename T>
__device__ __forceinline__ float ex_dot(const T* __restrict__ w, const float* __restrict__ a, int K, int lane, bool vectors) {
    float acc = 0.f;
    if (vectors) {
        constexpr int V = 16 / sizeof(T);
        typedef __attribute__((ext_vector_type(V))) T vec;
        for (int c = lane * V; c < K; c += KA_WAVE * V) {
            const vec x = *reinterpret_cast<const vec*>(w + c);
#pragma unroll
            for (int e = 0; e < V; ++e) acc = fmaf(ka_to_float(x[e]), a[c + e], acc);
        }
    } else {
        for (int c = lane; c < K; c += KA_WAVE) acc = fmaf(ka_to_float(w[c]), a[c], acc);
    }
    return ka_wave_sum(acc);
}

template <typename T>
__global__ void __launch_bounds__(256)
experts_linear_kernel(const T* __restrict__ a, long a_stride, int a_div, const T* __restrict__ W, const int* __restrict__ chosen,
                      int E, int N, int K, int act, void* __restrict__ out, long out_stride, int out_f32) {
    extern __shared__ float row[];
    const int p = blockIdx.y;
    const int e = chosen[p];
    if (e < 0 || e >= E) return;
    const T* ap = a + (size_t)(p / a_div) * a_stride;
    for (int c = threadIdx.x; c < K; c += blockDim.x) row[c] = ka_to_float(ap[c]);
    __syncthreads();
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const bool gated = ka_act_gated(act);
    const int n_out = gated ? N / 2 : N;
    const T* We = W + (size_t)e * N * K;
    const bool vectors = K % (16 / sizeof(T)) == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0;
    for (int q = wave; q < EX_COLS; q += 4) {
        const int j = blockIdx.x * EX_COLS + q;
        if (j >= n_out) break;
        float y;
        if (gated) {
            const float g = ex_dot(We + (size_t)(2 * j) * K, row, K, lane, vectors);
            const float v = ex_dot(We + (size_t)(2 * j + 1) * K, row, K, lane, vectors);
            y = ka_activate(act, g) * v;
        } else {
            y = ex_dot(We + (size_t)j * K, row, K, lane, vectors);
            if (ka_act_base(act)) y = ka_activate(act, y);
        }
        if (lane == 0) {
            if (out_f32) reinterpret_cast<float*>(out)[(size_t)p * out_stride + j] = y;
            else reinterpret_cast<T*>(out)[(size_t)p * out_stride + j] = ka_from_float<T>(y);
        }
    }
}

KA_API int ka_experts_linear(const void* a, long a_stride, int a_div, const void* W, int dtype, const int* chosen, int n_pairs,
                             int E, int N, int K, int act, void* out, long out_stride, int out_f32, hipStream_t stream) {
    const char* who = "ka_experts_linear";
    KA_CHECK(n_pairs >= 0 && E > 0 && N > 0 && K > 0 && a_div > 0, "%s: bad sizes", who);
    KA_CHECK(ka_act_known(act) && (!ka_act_gated(act) || N % 2 == 0), "%s: unknown activation %d, or a gated linear of %d rows", who, act, N);
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "%s: unsupported dtype %d", who, dtype);
    KA_CHECK(a_stride >= K && out_stride >= ka_act_outputs(act, N), "%s: a row stride is smaller than its row", who);
    KA_CHECK((size_t)K * sizeof(float) <= 64 * 1024, "%s: rows of %d numbers do not fit in LDS", who, K);
    KA_CHECK(n_pairs <= 65535, "%s: too many pairs %d", who, n_pairs);
    if (n_pairs == 0) return 0;
    dim3 grid((ka_act_outputs(act, N) + EX_COLS - 1) / EX_COLS, n_pairs);
    const size_t lds = (size_t)K * sizeof(float);
    if (dtype == KA_F32)
        hipLaunchKernelGGL(experts_linear_kernel<float>, grid, dim3(256), lds, stream, (const float*)a, a_stride, a_div, (const float*)W,
                           chosen, E, N, K, act, out, out_stride, out_f32);
    else
        hipLaunchKernelGGL(experts_linear_kernel<bf16_t>, grid, dim3(256), lds, stream, (const bf16_t*)a, a_stride, a_div, (const bf16_t*)W,
                           chosen, E, N, K, act, out, out_stride, out_f32);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The weighted sum: out[t] (=, or += if accumulate) sum_k weights[t, k] * (chosen[t, k] < E ? y[t * top + k] : h[t])
//     + sigmoid(shared_gate[t]) * shared[t]       (shared optional; without a gate its weight is 1).
// y fp32 [n top, dim], h of type T (the experts' input), shared fp32 [n, dim], out fp32 [n, dim].
// ----------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
experts_combine_kernel(const float* __restrict__ y, const T* __restrict__ h, long h_stride, const int* __restrict__ chosen,
                       const float* __restrict__ weights, int top, int E, const float* __restrict__ shared,
                       const float* __restrict__ shared_gate, long gate_stride, float* __restrict__ out, int dim, int accumulate) {
    const int t = blockIdx.x;
    const float sg = shared ? (shared_gate ? 1.0f / (1.0f + expf(-shared_gate[(size_t)t * gate_stride])) : 1.f) : 0.f;
    for (int c = threadIdx.x; c < dim; c += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = chosen[(size_t)t * top + k];
            const float v = e < E ? y[((size_t)t * top + k) * dim + c] : ka_to_float(h[(size_t)t * h_stride + c]);
            acc = fmaf(weights[(size_t)t * top + k], v, acc);
        }
        if (shared) acc = fmaf(sg, shared[(size_t)t * dim + c], acc);
        float* o = out + (size_t)t * dim + c;
        *o = accumulate ? *o + acc : acc;
    }
}

KA_API int ka_experts_combine(const float* y, const void* h, long h_stride, int dtype, const int* chosen, const float* weights, int n,
                              int top, int E, const float* shared, const float* shared_gate, long gate_stride, float* out, int dim,
                              int accumulate, hipStream_t stream) {
    KA_CHECK(n >= 0 && top > 0 && dim > 0 && h_stride >= dim, "ka_experts_combine: bad sizes");
    KA_CHECK(dtype == KA_F32 || dtype == KA_BF16, "ka_experts_combine: unsupported dtype %d", dtype);
    if (n == 0) return 0;
    if (dtype == KA_F32)
        hipLaunchKernelGGL(experts_combine_kernel<float>, dim3(n), dim3(256), 0, stream, y, (const float*)h, h_stride, chosen, weights, top,
                           E, shared, shared_gate, gate_stride, out, dim, accumulate);
    else
        hipLaunchKernelGGL(experts_combine_kernel<bf16_t>, dim3(n), dim3(256), 0, stream, y, (const bf16_t*)h, h_stride, chosen, weights,
                           top, E, shared, shared_gate, gate_stride, out, dim, accumulate);
    KA_LAUNCH_CHECK();
    return 0;
}

// ----------------------------------------------------------------------------
// The pairs listed by expert, for kernels that take an expert's pairs together: one workgroup counts the pairs of
// every expert, lays the experts' runs one behind the other, each run starting on a multiple of `tile` rows of the
// list, and fills them. sorted [capacity] holds pair numbers (-1 in the unused rows of a run's last tile);
// tile_expert [capacity / tile] the expert of every tile of the list (-1 behind the last run). Pairs of identity experts
// are in no run. Which row of its run a pair gets depends on the order the threads arrive in; nothing computed from the
// list depends on it (every pair's result is computed from its own row alone).
// capacity >= n_pairs rounded up to tiles + E tiles.
// ----------------------------------------------------------------------------
__global__ void __launch_bounds__(1024)
experts_sort_kernel(const int* __restrict__ chosen, int n_pairs, int E, int tile, int capacity, int* __restrict__ sorted,
                    int* __restrict__ tile_expert) {
    __shared__ int count[EX_MAX_OUTPUTS];
    __shared__ int start[EX_MAX_OUTPUTS + 1];
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) count[e] = 0;
    for (int i = tid; i < capacity; i += blockDim.x) sorted[i] = -1;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < E) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) {
            start[e] = at;
            at += (count[e] + tile - 1) / tile * tile;
        }
        start[E] = at;
    }
    __syncthreads();
    const int tiles = capacity / tile;
    for (int i = tid; i < tiles; i += blockDim.x) {
        // the expert whose run holds row i * tile: the last one that starts at or before it and is not empty there
        int e_of = -1;
        const int at = i * tile;
        if (at < start[E]) {
            int lo = 0, hi = E - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) / 2;
                if (start[mid] <= at) lo = mid; else hi = mid - 1;
            }
            e_of = lo;
        }
        tile_expert[i] = e_of;
    }
    for (int e = tid; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = tid; p < n_pairs; p += blockDim.x) {
        const int e = chosen[p];
        if (e >= 0 && e < E) sorted[start[e] + atomicAdd(&count[e], 1)] = p;
    }
}

KA_API int ka_experts_sort(const int* chosen, int n_pairs, int E, int tile, int capacity, int* sorted, int* tile_expert,
                           hipStream_t stream) {
    KA_CHECK(n_pairs >= 0 && E > 0 && E <= EX_MAX_OUTPUTS && tile > 0 && capacity % tile == 0, "ka_experts_sort: bad sizes");
    // (every expert's run may end in a tile that is not full)
    KA_CHECK((long)capacity >= (long)n_pairs + (long)E * (tile - 1), "ka_experts_sort: a list of %d rows is too short", capacity);
    hipLaunchKernelGGL(experts_sort_kernel, dim3(1), dim3(1024), 0, stream, chosen, n_pairs, E, tile, capacity, sorted, tile_expert);
    KA_LAUNCH_CHECK();
    return 0;
}
