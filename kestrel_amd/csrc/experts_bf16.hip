// The linears of routed experts on the matrix cores (bf16): the pairs (token, choice) of a step come listed by expert, in
// runs that start on multiples of 64 rows of the list (ka_experts_sort), and a workgroup multiplies one tile of 64 list
// rows by 128 rows of its expert's weights: out[row] = act(a[row'] W_e^T).
//
//  * the first linear gathers: list row i holds pair p = sorted[i] (-1: an unused row), whose input is row p / gather_div
//    of `a`; its output goes to row i of `out` (the hidden rows stay in list order);
//  * the second linear scatters: its input is row i of `a`, its output goes to row p of `out`;
//  * gated (KA_ACT_GATED): weight rows 2j and 2j + 1 are gate and value of output j, as in every gated linear here.
//
// Both operands are rows that are contiguous along k, which is how v_mfma_f32_32x32x16_bf16 wants them: a lane loads 16
// bytes of two weight rows and of two activation rows per step straight from memory (a wave owns 64 weight rows and both
// halves of the tile's 64 list rows, so four loads feed four products; the activation rows are shared with the other
// waves through the first-level cache). The weights are the row operand: a lane ends with outputs of ONE list row, four
// neighbours at a time, so the pair of a gated output meets in a lane's registers.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 eb_bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 eb_bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 eb_bf16x4;
typedef __attribute__((ext_vector_type(16))) float eb_floatx16;

constexpr int EB_ROWS = 64;      // list rows a workgroup (and a tile of the list)
constexpr int EB_COLS = 256;     // weight rows a workgroup: 64 a wave

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
    const int p0 = sorted[i0 + col], p1 = sorted[i0 + 32 + col];
    // rows past the end, and unused rows of the list, are clamped for the loads and not stored
    const bf16_t* wp0 = W + ((size_t)e * N + min(o0 + col, N - 1)) * K + half * 8;
    const bf16_t* wp1 = W + ((size_t)e * N + min(o0 + 32 + col, N - 1)) * K + half * 8;
    const long r0 = gather_div > 0 ? (long)max(p0, 0) / gather_div : (long)i0 + col;
    const long r1 = gather_div > 0 ? (long)max(p1, 0) / gather_div : (long)i0 + 32 + col;
    const bf16_t* ap0 = a + r0 * lda + half * 8;
    const bf16_t* ap1 = a + r1 * lda + half * 8;
    // acc[wb][rb]: weight rows o0 + 32 wb .., list rows i0 + 32 rb ..
    eb_floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[0][0][i] = acc[0][1][i] = acc[1][0][i] = acc[1][1][i] = 0.f;
#pragma unroll 2
    for (int kk = 0; kk < K; kk += 16) {
        const eb_bf16x8 w0 = *reinterpret_cast<const eb_bf16x8*>(wp0 + kk);
        const eb_bf16x8 w1 = *reinterpret_cast<const eb_bf16x8*>(wp1 + kk);
        const eb_bf16x8 a0 = *reinterpret_cast<const eb_bf16x8*>(ap0 + kk);
        const eb_bf16x8 a1 = *reinterpret_cast<const eb_bf16x8*>(ap1 + kk);
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w0, a0, acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w0, a1, acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1, a0, acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1, a1, acc[1][1], 0, 0, 0);
    }
    const bool gated = ka_act_gated(act);
#pragma unroll
    for (int both = 0; both < 4; ++both) {
        const int blk = both & 1, wb = both >> 1;
        const int p = blk ? p1 : p0;
        if (p < 0) continue;
        const eb_floatx16& acc_here = acc[wb][blk];
        const long row = scatter ? (long)p : (long)i0 + blk * 32 + col;
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
    hipLaunchKernelGGL(experts_gemm_kernel, grid, dim3(256), 0, stream, (const bf16_t*)a, lda, gather_div, (const bf16_t*)W, sorted,
                       tile_expert, N, K, act, out, ldo, scatter, out_f32);
    KA_LAUNCH_CHECK();
    return 0;
}
