// Matrix products out[M, N] = x[M, K] * w[N, K]^T (+ bias[N]).
//
// Both operands are row-major with K contiguous, which is how activations and
// nn.Linear-layout weights are stored.  This file holds the general kernel: a 64x64
// tile, 256 threads with a 4x4 micro-tile each, products and sums in true 32-bit
// (v_fma_f32; no matrix-core instruction of reduced precision).  It is the matrix
// product of the 32-bit path and the fallback of the bfloat16 path for shapes that
// the matrix-core kernels refuse.  The sum over K runs in one fixed order for every
// output element, whatever M is, so a row's result does not depend on the batch.
#include "common.h"

#define GT_M 64
#define GT_N 64
#define GT_K 16

template <typename TIn, typename TOut>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const TIn* __restrict__ x, const TIn* __restrict__ w,
                                                        const void* __restrict__ bias, int bias_f32,
                                                        TOut* __restrict__ out, int M, int N, int K,
                                                        int ldx, int ldo) {
    __shared__ float xs[GT_K][GT_M + 4];
    __shared__ float ws[GT_K][GT_N + 4];
    const int m0 = blockIdx.y * GT_M, n0 = blockIdx.x * GT_N;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    // loaders: 64 rows x 16 k per operand = 1024 elements, 4 per thread
    const int lrow = threadIdx.x / 4;         // 0..63
    const int lk = (threadIdx.x % 4) * 4;     // 0,4,8,12
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GT_K) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            const int m = m0 + lrow, n = n0 + lrow;
            xs[lk + i][lrow] = (m < M && k < K) ? to_float(x[(size_t)m * ldx + k]) : 0.f;
            ws[lk + i][lrow] = (n < N && k < K) ? to_float(w[(size_t)n * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GT_K; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += load_vec(bias, bias_f32, n);
            out[(size_t)m * ldo + n] = from_float<TOut>(v);
        }
    }
}

// dtype: of x and w.  out_f32: write 32-bit results (logits) whatever the input dtype.
extern "C" int tl_gemm_general(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                               int M, int N, int K, int ldx, int ldo, int dtype, int out_f32,
                               hipStream_t stream) {
    TL_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldo >= N, "gemm: bad sizes M=%d N=%d K=%d ldx=%d ldo=%d", M, N, K, ldx, ldo);
    if (M == 0) return TL_OK;
    dim3 grid((N + GT_N - 1) / GT_N, (M + GT_M - 1) / GT_M), block(256);
    if (dtype == TL_DT_F32)
        gemm_tile_kernel<float, float><<<grid, block, 0, stream>>>((const float*)x, (const float*)w, bias, bias_f32, (float*)out, M, N, K, ldx, ldo);
    else if (dtype == TL_DT_BF16 && out_f32)
        gemm_tile_kernel<bf16_t, float><<<grid, block, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (float*)out, M, N, K, ldx, ldo);
    else if (dtype == TL_DT_BF16)
        gemm_tile_kernel<bf16_t, bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (bf16_t*)out, M, N, K, ldx, ldo);
    else TL_REQUIRE(false, "gemm: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("gemm_general");
    return TL_OK;
}
