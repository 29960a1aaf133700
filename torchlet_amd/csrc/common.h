// Shared device helpers of the torchlet_amd kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// ---------------------------------------------------------------- element types
// bfloat16 is carried as its 16 raw bits; every kernel widens to float on load and
// rounds to nearest-even on store.
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(((uint32_t)v.bits) << 16); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) {
    // gfx950 converts in hardware (v_cvt_pk_bf16_f32): round to nearest, ties to even, NaN kept
    const __bf16 h = (__bf16)v;
    bf16_t r;
    __builtin_memcpy(&r.bits, &h, sizeof(r.bits));
    return r;
}

// A vector (norm weight, bias) is stored either as bfloat16 or as float; read element i.
__device__ __forceinline__ float load_vec(const void* p, int is_f32, int i) {
    return is_f32 ? ((const float*)p)[i] : to_float(((const bf16_t*)p)[i]);
}

// ---------------------------------------------------------------- reductions
#define TL_WAVE 64

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = TL_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, TL_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = TL_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, TL_WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `red` points to at least 16 floats of shared memory.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
    const int nw = (blockDim.x + TL_WAVE - 1) / TL_WAVE;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}

// ---------------------------------------------------------------- host side
// Every entry point returns 0 on success, else an error code; the text of the last
// error of the calling thread is read with tl_last_error().
#define TL_OK 0
#define TL_ERR_ARG 1
#define TL_ERR_HIP 2

#include <stdarg.h>
#include <stdio.h>

// Each shared library is one translation unit and carries its own error text.
static thread_local char tl_error_text[512];

static inline void tl_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(tl_error_text, sizeof(tl_error_text), fmt, ap);
    va_end(ap);
}

extern "C" const char* tl_last_error() { return tl_error_text; }

#define TL_REQUIRE(cond, ...)                 \
    do {                                      \
        if (!(cond)) {                        \
            tl_set_error(__VA_ARGS__);        \
            return TL_ERR_ARG;                \
        }                                     \
    } while (0)

#define TL_CHECK_LAUNCH(name)                                                    \
    do {                                                                         \
        hipError_t e_ = hipGetLastError();                                       \
        if (e_ != hipSuccess) {                                                  \
            tl_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
            return TL_ERR_HIP;                                                   \
        }                                                                        \
    } while (0)

#define TL_DT_F32 0
#define TL_DT_BF16 1
