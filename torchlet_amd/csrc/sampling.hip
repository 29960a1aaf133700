// Sampling from logits: greedy (arg max, lowest index on ties) and temperature sampling
// by the Gumbel-max rule, in two stages: many work-groups scan a row, one wave picks.
//
// Temperature t > 0: the token is argmax_i(logit_i / t + g_i) with g_i = -log(-log(u_i)),
// which is an exact draw from softmax(logits / t).  u_i comes from a counter-based hash
// of the row's 32-bit key and the index i, so a draw depends on nothing but (key, logits):
// not on the batch, the row's place in it, or the grid.
#include "common.h"
#include "sampling.h"
#include <mutex>

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

// One row's candidate: the larger value wins, the lower index on ties.
__device__ __forceinline__ void keep_better(float& best, int& besti, float v, int i) {
    if (v > best || (v == best && i < besti)) { best = v; besti = i; }
}

__device__ __forceinline__ void wave_best(float& best, int& besti) {
#pragma unroll
    for (int o = TL_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, TL_WAVE);
        const int oi = __shfl_xor(besti, o, TL_WAVE);
        keep_better(best, besti, ov, oi);
    }
}

// Stage 1: work-group (chunk, row) scans columns [chunk * per, (chunk + 1) * per) of its row and
// leaves its candidate in part_v / part_i [row, chunk].  A row of a large vocabulary is spread
// over many work-groups, so the scan is as wide as the machine and not as long as the row.
#define SAMPLE_THREADS 256
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_scan_kernel(const float* __restrict__ logits, int vocab, int ld, int per,
                                                                     const float* __restrict__ temperature,
                                                                     const int* __restrict__ keys,
                                                                     float* __restrict__ part_v, int* __restrict__ part_i) {
    __shared__ float bv[SAMPLE_THREADS / TL_WAVE];
    __shared__ int bi[SAMPLE_THREADS / TL_WAVE];
    const int chunk = blockIdx.x, row = blockIdx.y;
    const float* x = logits + (size_t)row * ld;
    const float t = temperature ? temperature[row] : 0.f;
    const uint32_t key = keys ? (uint32_t)keys[row] : 0u;
    const int end = min(vocab, (chunk + 1) * per);
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int i = chunk * per + threadIdx.x; i < end; i += SAMPLE_THREADS) {
        float v = x[i];
        if (t > 0.f) v = v / t + gumbel(key, (uint32_t)i);
        if (v > best) { best = v; besti = i; }        // strided scan: earlier i wins ties
    }
    wave_best(best, besti);
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    if (lane == 0) { bv[wave] = best; bi[wave] = besti; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < SAMPLE_THREADS / TL_WAVE; ++w) keep_better(best, besti, bv[w], bi[w]);
        part_v[(size_t)row * gridDim.x + chunk] = best;
        part_i[(size_t)row * gridDim.x + chunk] = besti;
    }
}

// Stage 2: one wave per row picks among the chunks' candidates.
__global__ __launch_bounds__(TL_WAVE) void sample_pick_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i,
                                                              int chunks, int vocab, int* __restrict__ out) {
    const int row = blockIdx.x;
    float best = -INFINITY;
    int besti = 0x7fffffff;
    for (int c = threadIdx.x; c < chunks; c += TL_WAVE)
        keep_better(best, besti, part_v[(size_t)row * chunks + c], part_i[(size_t)row * chunks + c]);
    wave_best(best, besti);
    if (threadIdx.x == 0) out[row] = besti < vocab ? besti : 0;
}

// Chunks a row of `vocab` columns is scanned in: about a thousand columns each, 128 at most.
extern "C" int tl_sample_chunks(int vocab) {
    const int c = (vocab + 1023) / 1024;
    return c < 1 ? 1 : (c > TL_SAMPLE_MAX_CHUNKS ? TL_SAMPLE_MAX_CHUNKS : c);
}

// Both stages; `candidates` holds rows * chunks floats, then rows * chunks ints.
static int launch_sample(const void* logits, int rows, int vocab, int ld, const void* temperature, const void* keys,
                         void* out, void* candidates, hipStream_t stream) {
    const int chunks = tl_sample_chunks(vocab);
    const int per = (vocab + chunks - 1) / chunks;
    float* part_v = (float*)candidates;
    int* part_i = (int*)candidates + (size_t)rows * chunks;
    sample_scan_kernel<<<dim3(chunks, rows), dim3(SAMPLE_THREADS), 0, stream>>>((const float*)logits, vocab, ld, per,
        (const float*)temperature, (const int*)keys, part_v, part_i);
    TL_CHECK_LAUNCH("sample_scan");
    sample_pick_kernel<<<dim3(rows), dim3(TL_WAVE), 0, stream>>>(part_v, part_i, chunks, vocab, (int*)out);
    TL_CHECK_LAUNCH("sample_pick");
    return TL_OK;
}

// temperature: float[rows] or null (all greedy); keys: int32[rows] bit patterns or null.
// scratch: rows * tl_sample_chunks(vocab) * 8 bytes, 4-byte aligned.
extern "C" int tl_sample(const void* logits, int rows, int vocab, int ld, const void* temperature,
                         const void* keys, void* out, void* scratch, hipStream_t stream) {
    TL_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample: bad sizes rows=%d vocab=%d ld=%d", rows, vocab, ld);
    TL_REQUIRE(scratch != nullptr || rows == 0, "sample: no scratch buffer");
    if (rows == 0) return TL_OK;
    return launch_sample(logits, rows, vocab, ld, temperature, keys, out, scratch, stream);
}

// ---------------------------------------------------------------- the entry point that allocates nothing
// The candidates' array of tl_sample_static, held by the library on every GPU it runs on.  In host code
// this name is only a stand-in for the symbol: the array's address on a GPU comes from
// hipGetSymbolAddress, asked once per device with that device current, and is what kernels are given.
static __device__ __align__(256) unsigned char scratch[(size_t)TL_SAMPLE_STATIC_MAX_ROWS * TL_SAMPLE_MAX_CHUNKS * 8];

#define TL_MAX_DEVICES 64
static void* scratch_of_device[TL_MAX_DEVICES];      // null: not asked for yet
static std::mutex scratch_mutex;

// The address of `scratch` on the device that is current in this thread.
static int scratch_here(void** address) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) {
        tl_set_error("sample_static: hipGetDevice failed: %s", hipGetErrorString(e));
        return TL_ERR_HIP;
    }
    TL_REQUIRE(device >= 0 && device < TL_MAX_DEVICES, "sample_static: device %d is beyond the %d this library keeps track of",
               device, TL_MAX_DEVICES);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_of_device[device] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            tl_set_error("sample_static: hipGetSymbolAddress failed on device %d: %s", device, hipGetErrorString(e));
            return TL_ERR_HIP;
        }
        scratch_of_device[device] = ptr;
    }
    *address = scratch_of_device[device];
    return TL_OK;
}

extern "C" int tl_sample_static(const void* logits, int rows, int vocab, int ld, const void* temperature,
                                const void* keys, void* out, hipStream_t stream) {
    TL_REQUIRE(rows >= 0 && vocab > 0 && ld >= vocab, "sample_static: bad sizes rows=%d vocab=%d ld=%d", rows, vocab, ld);
    TL_REQUIRE(rows <= TL_SAMPLE_STATIC_MAX_ROWS, "sample_static: %d rows, but the library's own array holds the candidates of %d at most",
               rows, TL_SAMPLE_STATIC_MAX_ROWS);
    if (rows == 0) return TL_OK;
    TL_REQUIRE(logits != nullptr && out != nullptr, "sample_static: logits and out must be given");
    void* ptr = nullptr;
    const int rc = scratch_here(&ptr);
    if (rc != TL_OK) return rc;
    return launch_sample(logits, rows, vocab, ld, temperature, keys, out, ptr, stream);
}
