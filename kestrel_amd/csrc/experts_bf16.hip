// The linears of routed experts on the matrix cores (bf16): the pairs (token, choice) of a step come listed by expert, in
// runs that start on multiples of 128 rows of the list (ka_experts_sort), and a workgroup multiplies one tile of 128 list
// rows by 256 rows of its expert's weights: out[row] = act(a[row'] W_e^T).
//
//  * the first linear gathers: list row i holds pair p = sorted[i] (-1: an unused row), whose input is row p / gather_div
//    of `a`; its output goes to row i of `out` (the hidden rows stay in list order);
//  * the second linear scatters: its input is row i of `a`, its output goes to row p of `out`;
//  * gated (KA_ACT_GATED): weight rows 2j and 2j + 1 are gate and value of output j, as in every gated linear here.
//
// Both operands are rows that are contiguous along k, which is how v_mfma_f32_32x32x16_bf16 wants them: a lane loads 64
// bytes in a row of two weight rows and of four activation rows per slab of 64 channels, straight from memory (a wave
// owns 64 weight rows and all of the tile's 128 list rows: 24 loads feed 32 products; the activation rows are shared
// with the other waves through the first-level cache, and a weight row's line is used up by the lane pair that asked). The weights are the row operand: a lane ends with outputs of ONE list row, four
// neighbours at a time, so the pair of a gated output meets in a lane's registers.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 eb_bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 eb_bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 eb_bf16x4;
typedef __attribute__((ext_vector_type(16))) float eb_floatx16;

constexpr int EB_ROWS = 128;     // list rows a workgroup (and a tile of the list): four blocks of 32
constexpr int EB_COLS = 256;     // weight rows a workgroup: 64 a wave, two blocks of 32
constexpr int EB_SLAB = 64;      // channels of k a lane's loads cover at a time: with its partner lane a whole 128-byte line

__global__ void __launch_bounds__(256)
experts_gemm_kernel(const bf16_t* __restrict__ a, long lda, int gather_div, const bf16_t* __restrict__ W, const int* __restrict__ sorted,
                    const int* __restrict__ tile_expert, int N, int K, int act, void* __restrict__ out, long ldo, int scatter,
                    int out_f32) {
    const int tile = blockIdx.y;
    const int e = tile_expert[tile];
    if (e < 0) return;                                   // (the unused end of the list)
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int col = lane % 32, half = lane / 32;
    const int o0 = blockIdx.x * EB_COLS + wave * 64;
    if (o0 >= N) return;                                 // (a whole wave; the kernel has no barrier)
    const int i0 = tile * EB_ROWS;
    int pr[4];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) pr[rb] = sorted[i0 + rb * 32 + col];
    // rows past the end, and unused rows of the list, are clamped for the loads and not stored
    const bf16_t* wp[2];
#pragma unroll
    for (int wb = 0; wb < 2; ++wb) wp[wb] = W + ((size_t)e * N + min(o0 + wb * 32 + col, N - 1)) * K;
    const bf16_t* ap[4];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
        ap[rb] = a + (gather_div > 0 ? (long)max(pr[rb], 0) / gather_div : (long)i0 + rb * 32 + col) * lda;
    // acc[wb][rb]: weight rows o0 + 32 wb .., list rows i0 + 32 rb ..
    eb_floatx16 acc[2][4];
#pragma unroll
    for (int wb = 0; wb < 2; ++wb)
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[wb][rb][i] = 0.f;
    // Slabs of 64 channels: a lane reads the 32 channels [32 half, 32 half + 32) of its rows, 64 bytes in a row, and feeds
    // them to four products, eight channels each. Which channels meet in a product does not matter as long as both
    // operands agree, and they do: piece m of half h is the channels 32 h + 8 m .. + 7 of the slab for both.
    // (the next slab's loads are asked for before the products of this one: a wave has its SIMD to itself, and nothing
    // else would hide their way from memory)
    int kk = 0;
    eb_bf16x8 w[2][4], x[4][4];
    auto load = [&](int at, eb_bf16x8 (&wn)[2][4], eb_bf16x8 (&xn)[4][4]) {
#pragma unroll
        for (int wb = 0; wb < 2; ++wb)
#pragma unroll
            for (int m = 0; m < 4; ++m) wn[wb][m] = *reinterpret_cast<const eb_bf16x8*>(wp[wb] + at + half * 32 + m * 8);
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int m = 0; m < 4; ++m) xn[rb][m] = *reinterpret_cast<const eb_bf16x8*>(ap[rb] + at + half * 32 + m * 8);
    };
    if (EB_SLAB <= K) load(0, w, x);
    for (; kk + EB_SLAB <= K; kk += EB_SLAB) {
        eb_bf16x8 wn[2][4], xn[4][4];
        const bool more = kk + 2 * EB_SLAB <= K;
        if (more) load(kk + EB_SLAB, wn, xn);
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int wb = 0; wb < 2; ++wb)
#pragma unroll
                for (int rb = 0; rb < 4; ++rb)
                    acc[wb][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w[wb][m], x[rb][m], acc[wb][rb], 0, 0, 0);
        if (more) {
#pragma unroll
            for (int m = 0; m < 4; ++m) {
#pragma unroll
                for (int wb = 0; wb < 2; ++wb) w[wb][m] = wn[wb][m];
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) x[rb][m] = xn[rb][m];
            }
        }
    }
    for (; kk < K; kk += 16) {                            // (what is left of a K that is no multiple of 64: steps of 16)
        eb_bf16x8 wt[2], xt[4];
#pragma unroll
        for (int wb = 0; wb < 2; ++wb) wt[wb] = *reinterpret_cast<const eb_bf16x8*>(wp[wb] + kk + half * 8);
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) xt[rb] = *reinterpret_cast<const eb_bf16x8*>(ap[rb] + kk + half * 8);
#pragma unroll
        for (int wb = 0; wb < 2; ++wb)
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) acc[wb][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wt[wb], xt[rb], acc[wb][rb], 0, 0, 0);
    }
    const bool gated = ka_act_gated(act);
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
        const int p = pr[rb];
        if (p < 0) continue;
        const long row = scatter ? (long)p : (long)i0 + rb * 32 + col;
#pragma unroll
        for (int wb = 0; wb < 2; ++wb) {
            const eb_floatx16& acc_here = acc[wb][rb];
            // register i: weight row o0 + 32 wb + (i / 4) * 8 + half * 4 + i % 4 of the lane's list row
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int o = o0 + wb * 32 + g4 * 8 + half * 4;
                if (gated) {
                    if (o + 3 < N) {
                        eb_bf16x2 y;
                        y[0] = (bf16_t)(ka_activate_fast(act, acc_here[g4 * 4]) * acc_here[g4 * 4 + 1]);
                        y[1] = (bf16_t)(ka_activate_fast(act, acc_here[g4 * 4 + 2]) * acc_here[g4 * 4 + 3]);
                        *reinterpret_cast<eb_bf16x2*>(reinterpret_cast<bf16_t*>(out) + row * ldo + o / 2) = y;
                    } else if (o + 1 < N) {
                        reinterpret_cast<bf16_t*>(out)[row * ldo + o / 2] = (bf16_t)(ka_activate_fast(act, acc_here[g4 * 4]) * acc_here[g4 * 4 + 1]);
                    }
                } else if (out_f32) {
                    float* op = reinterpret_cast<float*>(out) + row * ldo + o;
                    if (o + 3 < N) {
                        *reinterpret_cast<float4*>(op) = make_float4(acc_here[g4 * 4], acc_here[g4 * 4 + 1], acc_here[g4 * 4 + 2], acc_here[g4 * 4 + 3]);
                    } else {
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            if (o + x < N) op[x] = acc_here[g4 * 4 + x];
                    }
                } else {
                    bf16_t* op = reinterpret_cast<bf16_t*>(out) + row * ldo + o;
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        if (o + x < N) op[x] = (bf16_t)(ka_act_base(act) ? ka_activate_fast(act, acc_here[g4 * 4 + x]) : acc_here[g4 * 4 + x]);
                }
            }
        }
    }
}

// The same product with its operands staged through LDS, for K that is a multiple of 64: the workgroup's 256 threads fetch
// a slab of 64 channels of the tile's 128 list rows and 256 weight rows by whole 128-byte lines (eight lanes a row), once
// for all four waves, into registers while the slab before is multiplied, then into the other of two LDS buffers; a
// wave reads its operands from there, 16 bytes a lane (rows 144 bytes apart, so that the 16 lanes of a pass fall on all
// banks). One barrier a slab, which waits for LDS alone. Without it every wave fetched the tile's list rows for itself:
// 96 KB a slab through a compute unit's first-level cache where its products take 1,024 cycles.
constexpr int EB_PITCH = EB_SLAB + 8;                          // bf16 numbers from one LDS row to the next
constexpr int EB_STAGE = (EB_ROWS + EB_COLS) * EB_PITCH;       // numbers of one buffer: the list rows, then the weight rows

__global__ void __launch_bounds__(256)
experts_gemm_lds_kernel(const bf16_t* __restrict__ a, long lda, int gather_div, const bf16_t* __restrict__ W,
                        const int* __restrict__ sorted, const int* __restrict__ tile_expert, int N, int K, int act,
                        void* __restrict__ out, long ldo, int scatter, int out_f32) {
    extern __shared__ __attribute__((aligned(16))) bf16_t eb_lds[];
    const int tile = blockIdx.y;
    const int e = tile_expert[tile];
    if (e < 0) return;                                   // (the unused end of the list: the whole workgroup)
    const int tid = threadIdx.x;
    const int wave = tid / KA_WAVE, lane = tid % KA_WAVE;
    const int col = lane % 32, half = lane / 32;
    const int o0 = blockIdx.x * EB_COLS + wave * 64;
    const bool computes = o0 < N;
    const int i0 = tile * EB_ROWS;
    int pr[4];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) pr[rb] = sorted[i0 + rb * 32 + col];
    // what this thread fetches of every slab: piece tid % 8 (16 bytes) of the rows tid / 8 + 32 i: four list rows, eight
    // weight rows. Rows past the end, and unused rows of the list, are clamped for the loads and not stored.
    const int piece = tid % 8, row0 = tid / 8;
    const bf16_t* src[12];
    int dst[12];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = row0 + 32 * i;
        const int pair = sorted[i0 + r];
        src[i] = a + (gather_div > 0 ? (long)max(pair, 0) / gather_div : (long)i0 + r) * lda + piece * 8;
        dst[i] = r * EB_PITCH + piece * 8;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = row0 + 32 * i;
        src[4 + i] = W + ((size_t)e * N + min((int)blockIdx.x * EB_COLS + r, N - 1)) * K + piece * 8;
        dst[4 + i] = (EB_ROWS + r) * EB_PITCH + piece * 8;
    }
    eb_floatx16 acc[2][4];
#pragma unroll
    for (int wb = 0; wb < 2; ++wb)
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[wb][rb][i] = 0.f;
    eb_bf16x8 st[12];
    auto fetch = [&](int kk) {
#pragma unroll
        for (int i = 0; i < 12; ++i) st[i] = *reinterpret_cast<const eb_bf16x8*>(src[i] + kk);
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 12; ++i) *reinterpret_cast<eb_bf16x8*>(eb_lds + buf * EB_STAGE + dst[i]) = st[i];
    };
    auto lds_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(0xc07f);      // lgkmcnt(0), the other counters at their maximum
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    const int slabs = K / EB_SLAB;
    fetch(0);
    stage(0);
    lds_barrier();
    for (int sl = 0; sl < slabs; ++sl) {
        const int buf = sl & 1;
        if (sl + 1 < slabs) fetch((sl + 1) * EB_SLAB);
        if (computes) {
            const bf16_t* base = eb_lds + buf * EB_STAGE;
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                eb_bf16x8 w[2], x[4];
#pragma unroll
                for (int wb = 0; wb < 2; ++wb)
                    w[wb] = *reinterpret_cast<const eb_bf16x8*>(base + (EB_ROWS + wave * 64 + wb * 32 + col) * EB_PITCH + half * 32 + m * 8);
#pragma unroll
                for (int rb = 0; rb < 4; ++rb)
                    x[rb] = *reinterpret_cast<const eb_bf16x8*>(base + (rb * 32 + col) * EB_PITCH + half * 32 + m * 8);
#pragma unroll
                for (int wb = 0; wb < 2; ++wb)
#pragma unroll
                    for (int rb = 0; rb < 4; ++rb)
                        acc[wb][rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w[wb], x[rb], acc[wb][rb], 0, 0, 0);
            }
        }
        if (sl + 1 < slabs) stage(buf ^ 1);
        lds_barrier();
    }
    if (!computes) return;
    const bool gated = ka_act_gated(act);
#pragma unroll
    for (int rb = 0; rb < 4; ++rb) {
        const int p = pr[rb];
        if (p < 0) continue;
        const long row = scatter ? (long)p : (long)i0 + rb * 32 + col;
#pragma unroll
        for (int wb = 0; wb < 2; ++wb) {
            const eb_floatx16& acc_here = acc[wb][rb];
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int o = o0 + wb * 32 + g4 * 8 + half * 4;
                if (gated) {
                    if (o + 3 < N) {
                        eb_bf16x2 y;
                        y[0] = (bf16_t)(ka_activate_fast(act, acc_here[g4 * 4]) * acc_here[g4 * 4 + 1]);
                        y[1] = (bf16_t)(ka_activate_fast(act, acc_here[g4 * 4 + 2]) * acc_here[g4 * 4 + 3]);
                        *reinterpret_cast<eb_bf16x2*>(reinterpret_cast<bf16_t*>(out) + row * ldo + o / 2) = y;
                    } else if (o + 1 < N) {
                        reinterpret_cast<bf16_t*>(out)[row * ldo + o / 2] = (bf16_t)(ka_activate_fast(act, acc_here[g4 * 4]) * acc_here[g4 * 4 + 1]);
                    }
                } else if (out_f32) {
                    float* op = reinterpret_cast<float*>(out) + row * ldo + o;
                    if (o + 3 < N) {
                        *reinterpret_cast<float4*>(op) = make_float4(acc_here[g4 * 4], acc_here[g4 * 4 + 1], acc_here[g4 * 4 + 2], acc_here[g4 * 4 + 3]);
                    } else {
#pragma unroll
                        for (int x = 0; x < 4; ++x)
                            if (o + x < N) op[x] = acc_here[g4 * 4 + x];
                    }
                } else {
                    bf16_t* op = reinterpret_cast<bf16_t*>(out) + row * ldo + o;
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        if (o + x < N) op[x] = (bf16_t)(ka_act_base(act) ? ka_activate_fast(act, acc_here[g4 * 4 + x]) : acc_here[g4 * 4 + x]);
                }
            }
        }
    }
}

KA_API int ka_experts_gemm_tile() { return EB_ROWS; }

// Whether the kernel covers these sizes and this alignment.
KA_API int ka_experts_gemm_supported(long lda, int N, int K, long ldo, int act, int out_f32) {
    const int n_out = ka_act_outputs(act, N);
    return K > 0 && K % 16 == 0 && lda % 8 == 0 && N > 0 && (!ka_act_gated(act) || (N % 4 == 0 && ldo % 2 == 0 && !out_f32)) &&
           (!out_f32 || ldo % 4 == 0) && ldo >= n_out ? 1 : 0;
}

KA_API int ka_experts_gemm_bf16(const void* a, long lda, int gather_div, const void* W, const int* sorted, const int* tile_expert,
                                int n_tiles, int N, int K, int act, void* out, long ldo, int scatter, int out_f32,
                                hipStream_t stream) {
    const char* who = "ka_experts_gemm_bf16";
    KA_CHECK(n_tiles >= 0 && n_tiles <= 65535 && gather_div >= 0, "%s: bad sizes (%d tiles)", who, n_tiles);
    KA_CHECK(ka_act_known(act) && ka_experts_gemm_supported(lda, N, K, ldo, act, out_f32), "%s: sizes N=%d K=%d not covered", who, N, K);
    KA_CHECK((uintptr_t)a % 16 == 0 && (uintptr_t)W % 16 == 0 && (uintptr_t)out % 16 == 0, "%s: operands must be 16-byte aligned", who);
    if (n_tiles == 0) return 0;
    const dim3 grid((N + EB_COLS - 1) / EB_COLS, n_tiles);
    if (K % EB_SLAB == 0) {
        const size_t lds = 2 * (size_t)EB_STAGE * sizeof(bf16_t);
        static bool sized = false;
        if (!sized) {
            (void)hipFuncSetAttribute((const void*)experts_gemm_lds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            sized = true;
        }
        hipLaunchKernelGGL(experts_gemm_lds_kernel, grid, dim3(256), lds, stream, (const bf16_t*)a, lda, gather_div, (const bf16_t*)W,
                           sorted, tile_expert, N, K, act, out, ldo, scatter, out_f32);
    } else {
        hipLaunchKernelGGL(experts_gemm_kernel, grid, dim3(256), 0, stream, (const bf16_t*)a, lda, gather_div, (const bf16_t*)W, sorted,
                           tile_expert, N, K, act, out, ldo, scatter, out_f32);
    }
    KA_LAUNCH_CHECK();
    return 0;
}
