// A linear per head on the matrix cores: out[r, h, o] = sum_k a[r, h, k] * w[h, o, k] for every head h, with rows of `a`
// that hold heads of `a_head` channels (the first k of each are read) and rows of `out` that hold heads of `out_head`
// channels (the first n_out of each are written, the rest are left alone). bf16 in and out, sums in fp32. With `gate`
// (rows laid out as those of `out`, a row stride of their own) every output is multiplied by the sigmoid of its gate.
//
// What it is for: mixers that keep a low-rank latent per key and move the per-head up-projections to the query's side
// (every head's query times its own key matrix, every head's weighted sum of latents times its own value matrix). One
// launch takes all heads; a workgroup of four waves owns a tile of 64 rows x 64 outputs of one head, a wave a quadrant of
// 32 x 32 (v_mfma_f32_32x32x16_bf16). Both operands are rows that are contiguous along k, which is how the instruction
// wants them: a lane loads 16 bytes of its weight row and 16 bytes of its activation row per step, straight from memory
// (the tile's rows are re-read by the wave beside it out of the first-level cache; there is nothing to stage). The
// weights of the product are the row operand, the activations the column operand: a lane then ends with 16 outputs of
// ONE row of `out`, four neighbours at a time, which it stores as 8-byte pieces.
#include "ka_common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 hl_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 hl_bf16x4;
typedef __attribute__((ext_vector_type(16))) float hl_floatx16;

constexpr int HL_TILE = 64;

__global__ void __launch_bounds__(256)
heads_linear_kernel(const bf16_t* __restrict__ a, long lda, int a_head, const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                    long ldo, int out_head, int n, int n_out, int k, const bf16_t* __restrict__ gate, long ldg) {
    const int wave = threadIdx.x / KA_WAVE, lane = threadIdx.x % KA_WAVE;
    const int col = lane % 32, half = lane / 32;
    const int head = blockIdx.z;
    const int o0 = blockIdx.x * HL_TILE + (wave & 1) * 32, r0 = blockIdx.y * HL_TILE + (wave >> 1) * 32;
    if (o0 >= n_out || r0 >= n) return;                  // (a whole wave; the kernel has no barrier)
    // rows past the end are clamped for the loads and not stored
    const bf16_t* wp = w + ((size_t)head * n_out + min(o0 + col, n_out - 1)) * k + half * 8;
    const bf16_t* ap = a + (size_t)min(r0 + col, n - 1) * lda + (size_t)head * a_head + half * 8;
    hl_floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll 4
    for (int kk = 0; kk < k; kk += 16)
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const hl_bf16x8*>(wp + kk),
                                                      *reinterpret_cast<const hl_bf16x8*>(ap + kk), acc, 0, 0, 0);
    const int row = r0 + col;
    if (row >= n) return;
    // register i: output o0 + (i / 4) * 8 + half * 4 + i % 4 of the lane's row
    bf16_t* op = out + (size_t)row * ldo + (size_t)head * out_head;
    if (gate) {
        const bf16_t* gp = gate + (size_t)row * ldg + (size_t)head * out_head;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int o = o0 + (i / 4) * 8 + half * 4 + i % 4;
            if (o < n_out) acc[i] *= 1.0f / (1.0f + __expf(-(float)gp[o]));
        }
    }
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
        const int o = o0 + g4 * 8 + half * 4;
        if (o + 3 < n_out) {
            hl_bf16x4 y;
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = (bf16_t)acc[g4 * 4 + e];
            *reinterpret_cast<hl_bf16x4*>(op + o) = y;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (o + e < n_out) op[o + e] = (bf16_t)acc[g4 * 4 + e];
        }
    }
}

// Whether the kernel covers these sizes and this alignment.
KA_API int ka_heads_linear_supported(long lda, int a_head, long ldo, int out_head, int n_out, int k) {
    return k > 0 && k % 16 == 0 && a_head % 8 == 0 && lda % 8 == 0 && out_head % 4 == 0 && ldo % 4 == 0 && n_out > 0 &&
           a_head >= k && out_head >= n_out ? 1 : 0;
}

KA_API int ka_heads_linear_bf16(const void* a, long lda, int a_head, const void* w, void* out, long ldo, int out_head, int n,
                                int heads, int n_out, int k, const void* gate, long ldg, hipStream_t stream) {
    const char* who = "ka_heads_linear_bf16";
    KA_CHECK(n >= 0 && heads > 0 && heads <= 65535, "%s: bad sizes", who);
    KA_CHECK(ka_heads_linear_supported(lda, a_head, ldo, out_head, n_out, k), "%s: sizes k=%d n_out=%d heads of %d -> %d not covered", who, k, n_out, a_head, out_head);
    KA_CHECK(lda >= (long)heads * a_head && ldo >= (long)heads * out_head, "%s: rows shorter than their heads", who);
    KA_CHECK((uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 8 == 0, "%s: operands must be 16-byte aligned", who);
    if (n == 0) return 0;
    const dim3 grid((n_out + HL_TILE - 1) / HL_TILE, (n + HL_TILE - 1) / HL_TILE, heads);
    KA_CHECK(grid.y <= 65535, "%s: too many rows %d", who, n);
    hipLaunchKernelGGL(heads_linear_kernel, grid, dim3(256), 0, stream, (const bf16_t*)a, lda, a_head, (const bf16_t*)w,
                       (bf16_t*)out, ldo, out_head, n, n_out, k, (const bf16_t*)gate, ldg);
    KA_LAUNCH_CHECK();
    return 0;
}
