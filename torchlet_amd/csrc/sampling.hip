// Sampling from logits: greedy (arg max, lowest index on ties) and temperature sampling
// by the Gumbel-max rule, one block per row.
//
// Temperature t > 0: the token is argmax_i(logit_i / t + g_i) with g_i = -log(-log(u_i)),
// which is an exact draw from softmax(logits / t).  u_i comes from a counter-based hash
// of the row's 32-bit key and the index i, so a draw depends on nothing but (key, logits):
// not on the batch, the row's place in it, or the grid.
#include "common.h"

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352du;
    x ^= x >> 15; x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

__device__ __forceinline__ float gumbel(uint32_t key, uint32_t i) {
    const uint32_t r = mix32(mix32(key ^ i) + 0x9e3779b9u);
    const float u = ((float)(r >> 8) + 0.5f) * (1.0f / 16777216.0f);   // in (0, 1)
    return -logf(-logf(u));
}

__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits, int vocab, int ld,
                                                      const float* __restrict__ temperature,
                                                      const int* __restrict__ keys, int* __restrict__ out) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const int row = blockIdx.x;
    const float* x = logits + (size_t)row * ld;
    const float t = temperature ? temperature[row] : 0.f;
    const uint32_t key = keys ? (uint32_t)keys[row] : 0u;
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        float v = x[i];
        if (t > 0.f) v = v / t + gumbel(key, (uint32_t)i);
        if (v > best) { best = v; besti = i; }        // strided scan: earlier i wins ties
    }
#pragma unroll
    for (int o = TL_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, TL_WAVE);
        const int oi = __shfl_xor(besti, o, TL_WAVE);
        if (ov > best || (ov == best && oi < besti)) { best = ov; besti = oi; }
    }
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    if (lane == 0) { bv[wave] = best; bi[wave] = besti; }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nw = (blockDim.x + TL_WAVE - 1) / TL_WAVE;
        for (int w = 1; w < nw; ++w)
            if (bv[w] > best || (bv[w] == best && bi[w] < besti)) { best = bv[w]; besti = bi[w]; }
        out[row] = besti < vocab ? besti : 0;
    }
}

// temperature: float[rows] or null (all greedy); keys: int32[rows] bit patterns or null.
extern "C" int tl_sample(const void* logits, int rows, int vocab, int ld, const void* temperature,
                         const void* keys, void* out, hipStream_t stream) {
    TL_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%d", rows, vocab, ld);
    if (rows == 0) return TL_OK;
    sample_kernel<<<dim3(rows), dim3(1024), 0, stream>>>((const float*)logits, vocab, ld, (const float*)temperature,
                                                         (const int*)keys, (int*)out);
    TL_CHECK_LAUNCH("sample");
    return TL_OK;
}
