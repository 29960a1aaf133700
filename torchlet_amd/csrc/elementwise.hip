// Row-wise kernels: embedding gather, residual add + RMSNorm, rotary position
// encoding fused with the write of keys and values into cache pages, SwiGLU gate.
// Each is templated on the activation type (float or bfloat16); all arithmetic is float.
#include "common.h"

// ------------------------------------------------------------------ embedding
// out[t, :] = float(table[ids[t], :]) * scale; the residual stream is 32-bit.
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ out, int hidden, int vocab, float scale) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= vocab) id = 0;  // ids are checked on the host; never read out of bounds
    const T* src = table + (size_t)id * hidden;
    float* dst = out + (size_t)t * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) * scale;
}

extern "C" int tl_embedding(const void* ids, const void* table, int table_dtype, void* out,
                            int tokens, int hidden, int vocab, float scale, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0, "embedding: bad sizes tokens=%d hidden=%d vocab=%d", tokens, hidden, vocab);
    if (tokens == 0) return TL_OK;
    dim3 grid(tokens), block(256);
    if (table_dtype == TL_DT_F32)
        embedding_kernel<float><<<grid, block, 0, stream>>>((const int*)ids, (const float*)table, (float*)out, hidden, vocab, scale);
    else if (table_dtype == TL_DT_BF16)
        embedding_kernel<bf16_t><<<grid, block, 0, stream>>>((const int*)ids, (const bf16_t*)table, (float*)out, hidden, vocab, scale);
    else TL_REQUIRE(false, "embedding: unknown dtype %d", table_dtype);
    TL_CHECK_LAUNCH("embedding");
    return TL_OK;
}

// ------------------------------------------------------------------ add + RMSNorm
// One block per output row.  r = residual[row] (+ pending[row]); if `update`, r is
// written back to the residual; out = r * rsqrt(mean(r^2) + eps) * weight.
// `rows` (optional) selects the source row of each output row; then nothing is written back.
// `gain` multiplies the row's scale factor (1: the plain norm; a model with a factor on its logits puts it here).
// The pending branch output comes either as one [rows, hidden] tensor of the activation type
// (parts == 0) or as `parts` float slabs [parts, total_rows, hidden] of partial sums that are
// added up here (the split-K products write such slabs).
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const void* __restrict__ pending, int parts, size_t part_stride,
                                   const void* __restrict__ weight, int weight_f32, float eps, float gain,
                                   T* __restrict__ out, const int* __restrict__ rows, int hidden) {
    __shared__ float red[16];
    const int orow = blockIdx.x;
    const int srow = rows ? rows[orow] : orow;
    float* res = residual + (size_t)srow * hidden;
    const T* pen = (pending && parts == 0) ? (const T*)pending + (size_t)srow * hidden : nullptr;
    const float* pparts = (pending && parts > 0) ? (const float*)pending + (size_t)srow * hidden : nullptr;
    const bool update = (pending != nullptr) && (rows == nullptr);
    float ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float r = res[i];
        if (pen) r += to_float(pen[i]);
        if (pparts)
            for (int p = 0; p < parts; ++p) r += pparts[p * part_stride + i];
        if (update) res[i] = r;
        ss += r * r;
    }
    ss = block_sum(ss, red);
    const float inv = rsqrtf(ss / (float)hidden + eps) * gain;
    T* dst = out + (size_t)orow * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float r = res[i];
        if (!update) {
            if (pen) r += to_float(pen[i]);
            if (pparts)
                for (int p = 0; p < parts; ++p) r += pparts[p * part_stride + i];
        }
        dst[i] = from_float<T>(r * inv * load_vec(weight, weight_f32, i));
    }
}

// The same with every element of the row held in registers between the two passes: a thread
// owns IT groups of 4 contiguous elements, loaded with one 16-byte (float) or 8-byte
// (bfloat16) access each, so the row is read from memory once and the weight load overlaps
// the reduction.  Used when hidden % 4 == 0 and hidden <= 16 * blockDim.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 t = *(const float4*)p; v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4<bf16_t> {
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
        const uint2 t = *(const uint2*)p;
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
        uint2 t;
        t.x = (uint32_t)from_float<bf16_t>(v[0]).bits | ((uint32_t)from_float<bf16_t>(v[1]).bits << 16);
        t.y = (uint32_t)from_float<bf16_t>(v[2]).bits | ((uint32_t)from_float<bf16_t>(v[3]).bits << 16);
        *(uint2*)p = t;
    }
};

// r += the N slabs' four elements at src, src + stride, ...: all requested, then added in their order.
template <int N>
__device__ __forceinline__ void add_slabs(const float* src, size_t stride, float (&r)[4]) {
    float p[N][4];
#pragma unroll
    for (int u = 0; u < N; ++u) Vec4<float>::load(src + u * stride, p[u]);
#pragma unroll
    for (int u = 0; u < N; ++u)
#pragma unroll
        for (int v = 0; v < 4; ++v) r[v] += p[u][v];
}

template <typename T, int IT>
__global__ void add_rmsnorm_reg_kernel(float* __restrict__ residual, const void* __restrict__ pending, int parts, size_t part_stride,
                                       const void* __restrict__ weight, int weight_f32, float eps, float gain,
                                       T* __restrict__ out, const int* __restrict__ rows, int hidden) {
    __shared__ float red[16];
    const int orow = blockIdx.x;
    const int srow = rows ? rows[orow] : orow;
    float* res = residual + (size_t)srow * hidden;
    const T* pen = (pending && parts == 0) ? (const T*)pending + (size_t)srow * hidden : nullptr;
    const float* pparts = (pending && parts > 0) ? (const float*)pending + (size_t)srow * hidden : nullptr;
    const bool update = (pending != nullptr) && (rows == nullptr);
    float r[IT][4], wv[IT][4];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (it * blockDim.x + threadIdx.x) * 4;
        if (i < hidden) {
            Vec4<float>::load(res + i, r[it]);
            if (pen) {
                float p[4];
                Vec4<T>::load(pen + i, p);
#pragma unroll
                for (int v = 0; v < 4; ++v) r[it][v] += p[v];
            }
            if (pparts) {
                // four slabs at a time, all requested before the first is added (a loop over a count known
                // only at run time fetches one slab after the other: a trip to memory each); the sums are
                // added in the order of the slabs either way.  The last two or three slabs are a group as well
                // (three slabs, as for the matrices 5120 wide, were three trips).
                int q = 0;
                for (; q + 4 <= parts; q += 4) add_slabs<4>(pparts + q * part_stride + i, part_stride, r[it]);
                if (parts - q == 3) add_slabs<3>(pparts + q * part_stride + i, part_stride, r[it]);
                else if (parts - q == 2) add_slabs<2>(pparts + q * part_stride + i, part_stride, r[it]);
                else if (parts - q == 1) add_slabs<1>(pparts + q * part_stride + i, part_stride, r[it]);
            }
            if (weight_f32) Vec4<float>::load((const float*)weight + i, wv[it]);
            else Vec4<bf16_t>::load((const bf16_t*)weight + i, wv[it]);
#pragma unroll
            for (int v = 0; v < 4; ++v) ss += r[it][v] * r[it][v];
        }
    }
    if (update) {
#pragma unroll
        for (int it = 0; it < IT; ++it) {
            const int i = (it * blockDim.x + threadIdx.x) * 4;
            if (i < hidden) Vec4<float>::store(res + i, r[it]);
        }
    }
    ss = block_sum(ss, red);
    const float inv = rsqrtf(ss / (float)hidden + eps) * gain;
    T* dst = out + (size_t)orow * hidden;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int i = (it * blockDim.x + threadIdx.x) * 4;
        if (i < hidden) {
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) o[v] = r[it][v] * inv * wv[it][v];
            Vec4<T>::store(dst + i, o);
        }
    }
}

template <typename T>
static void launch_add_rmsnorm(float* residual, const void* pending, int parts, size_t part_stride, const void* weight,
                               int weight_f32, float eps, float gain, T* out, const int* rows, int out_rows, int hidden, hipStream_t stream) {
    const bool aligned = hidden % 4 == 0 && ((uintptr_t)residual % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                         ((uintptr_t)pending % 16) == 0 && ((uintptr_t)weight % 16) == 0;
    dim3 grid(out_rows);
    if (aligned && hidden <= 1024)
        add_rmsnorm_reg_kernel<T, 1><<<grid, 256, 0, stream>>>(residual, pending, parts, part_stride, weight, weight_f32, eps, gain, out, rows, hidden);
    else if (aligned && hidden <= 2048)
        add_rmsnorm_reg_kernel<T, 2><<<grid, 256, 0, stream>>>(residual, pending, parts, part_stride, weight, weight_f32, eps, gain, out, rows, hidden);
    else if (aligned && hidden <= 4096)
        add_rmsnorm_reg_kernel<T, 2><<<grid, 512, 0, stream>>>(residual, pending, parts, part_stride, weight, weight_f32, eps, gain, out, rows, hidden);
    else if (aligned && hidden <= 8192)
        add_rmsnorm_reg_kernel<T, 4><<<grid, 512, 0, stream>>>(residual, pending, parts, part_stride, weight, weight_f32, eps, gain, out, rows, hidden);
    else if (aligned && hidden <= 16384)
        add_rmsnorm_reg_kernel<T, 4><<<grid, 1024, 0, stream>>>(residual, pending, parts, part_stride, weight, weight_f32, eps, gain, out, rows, hidden);
    else
        add_rmsnorm_kernel<T><<<grid, hidden >= 2048 ? 512 : 256, 0, stream>>>(residual, pending, parts, part_stride, weight, weight_f32, eps, gain, out, rows, hidden);
}

// parts == 0: `pending` is [rows, hidden] of the activation type (or null); parts > 0: `pending` is
// float [parts, part_rows, hidden], slabs of partial sums to be added up.
extern "C" int tl_add_rmsnorm(void* residual, const void* pending, int parts, int part_rows, const void* weight,
                              int weight_f32, float eps, float gain, void* out, const void* rows, int out_rows, int hidden,
                              int act_dtype, hipStream_t stream) {
    TL_REQUIRE(parts >= 0 && parts <= 64, "add_rmsnorm: %d partial slabs", parts);
    const size_t part_stride = (size_t)part_rows * hidden;
    TL_REQUIRE(out_rows >= 0 && hidden > 0, "add_rmsnorm: bad sizes rows=%d hidden=%d", out_rows, hidden);
    if (out_rows == 0) return TL_OK;
    if (act_dtype == TL_DT_F32)
        launch_add_rmsnorm<float>((float*)residual, pending, parts, part_stride, weight, weight_f32, eps, gain, (float*)out, (const int*)rows, out_rows, hidden, stream);
    else if (act_dtype == TL_DT_BF16)
        launch_add_rmsnorm<bf16_t>((float*)residual, pending, parts, part_stride, weight, weight_f32, eps, gain, (bf16_t*)out, (const int*)rows, out_rows, hidden, stream);
    else TL_REQUIRE(false, "add_rmsnorm: unknown dtype %d", act_dtype);
    TL_CHECK_LAUNCH("add_rmsnorm");
    return TL_OK;
}

// ------------------------------------------------------------------ RoPE + cache write
// One wave per token and head.  Row layout of `qkv`: [q heads | k heads | v heads], each head
// `head_dim` wide, row stride `row_stride` elements.
//   * rotate (inv_freq != null): the first `rot_heads` heads (q, then k) are rotated in
//     place with the split-half pairing (j, j + head_dim/2) by angle = float(pos) * inv_freq[j];
//     with `pairs` the two elements of frequency j are the neighbours (2j, 2j + 1) instead.
//   * write (k_plane != null): rotated k and raw v of the token go to the page
//     block_table[token_req[t]][pos / page] at offset pos % page.  The key plane is
//     [pages, kv_heads, page, head_dim]; the value plane holds each page transposed,
//     [pages, kv_heads, head_dim, page], the layout the attention kernels read.  Page 0 is the
//     sentinel that empty block-table entries point to: a token whose page is 0 (a padding row of a
//     step of fixed shape) has its keys and values dropped, so nothing ever writes that page.
// One pair turned by its angle, in a fixed sequence of roundings (one product, one fused
// multiply-add per result), so that every kernel here gives the same bits for the same input.
__device__ __forceinline__ void rope_turn(float& x1, float& x2, float c, float sn) {
    const float y1 = __fmaf_rn(x1, c, -__fmul_rn(x2, sn));
    const float y2 = __fmaf_rn(x2, c, __fmul_rn(x1, sn));
    x1 = y1;
    x2 = y2;
}

#define ROPE_HEADS_PER_GROUP 4          // one wave per head, four heads per work-group
template <typename T>
__global__ __launch_bounds__(ROPE_HEADS_PER_GROUP * TL_WAVE)
void rope_cache_write_kernel(T* __restrict__ qkv, int row_stride, int q_heads, int kv_heads,
                             int head_dim, int rot_heads, const int* __restrict__ positions,
                             const float* __restrict__ inv_freq, const int* __restrict__ token_req,
                             const int* __restrict__ block_table, int bt_stride,
                             T* __restrict__ k_plane, T* __restrict__ v_plane, int page_size, int pairs, int pair_aligned,
                             const float* __restrict__ parts, int num_parts, size_t part_stride, int parts_ld,
                             const void* __restrict__ bias, int bias_f32) {
    // A wave owns one head of one token: a query head (rotated in place), a key head (rotated in
    // place and written to its page) or a value head (written to its page, transposed).  Each wave
    // takes the cosines and sines of its own pairs, so no wave waits for another.
    const int t = blockIdx.x;
    const int head = blockIdx.y * ROPE_HEADS_PER_GROUP + threadIdx.x / TL_WAVE;
    const int lane = threadIdx.x % TL_WAVE;
    const int heads = q_heads + kv_heads + (k_plane ? kv_heads : 0);
    if (head >= heads) return;
    const int pos = positions[t];
    const int half = head_dim / 2;
    T* x = qkv + (size_t)t * row_stride + (size_t)head * head_dim;
    T* dst = nullptr;                      // this head's place in the cache, if it has one
    if (k_plane && head >= q_heads) {
        const int page = block_table[(size_t)token_req[t] * bt_stride + pos / page_size];
        const int kvh = (head - q_heads) % kv_heads;
        const size_t base = ((size_t)page * kv_heads + kvh) * page_size * head_dim;
        if (page != 0)
            dst = head < q_heads + kv_heads ? k_plane + base + (size_t)(pos % page_size) * head_dim
                                            : v_plane + base + (pos % page_size);
    }
    // With `parts` the row does not come from qkv but is the sum of float slabs of partial sums
    // [num_parts][tokens, parts_ld] plus the bias (a projection that was split over K); the rotated
    // queries then go to qkv, keys and values to their pages only.
    auto element = [&](int i) -> float {
        if (!parts) return to_float(x[i]);
        const size_t col = (size_t)head * head_dim + i;
        float sum = bias ? load_vec(bias, bias_f32, col) : 0.f;
        const float* src = parts + (size_t)t * parts_ld + col;
        int p = 0;
        for (; p + 4 <= num_parts; p += 4) {       // four slabs requested before the first is added, in their order
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = src[(size_t)(p + u) * part_stride];
#pragma unroll
            for (int u = 0; u < 4; ++u) sum += v[u];
        }
        if (num_parts - p == 3) {                  // (and the last two or three)
            const float v0 = src[(size_t)p * part_stride], v1 = src[(size_t)(p + 1) * part_stride], v2 = src[(size_t)(p + 2) * part_stride];
            sum += v0; sum += v1; sum += v2;
        } else if (num_parts - p == 2) {
            const float v0 = src[(size_t)p * part_stride], v1 = src[(size_t)(p + 1) * part_stride];
            sum += v0; sum += v1;
        } else if (num_parts - p == 1) {
            sum += src[(size_t)p * part_stride];
        }
        return sum;
    };
    if (head >= q_heads + kv_heads) {      // value head: [head_dim, page] inside the page
        if (dst)
            for (int d = lane; d < head_dim; d += TL_WAVE) dst[(size_t)d * page_size] = from_float<T>(element(d));
        return;
    }
    const bool rotate = inv_freq && head < rot_heads;
    if (!rotate && !dst && !parts) return;
    if (pairs && pair_aligned && !parts) {
        // pair layout: the two elements of a frequency are one aligned load and one aligned store
        struct __attribute__((aligned(2 * sizeof(T)))) Two { T a, b; };
        for (int j = lane; j < half; j += TL_WAVE) {
            Two p = *(const Two*)(x + 2 * j);
            float x1 = to_float(p.a), x2 = to_float(p.b);
            if (rotate) {
                const float angle = (float)pos * inv_freq[j];
                rope_turn(x1, x2, cosf(angle), sinf(angle));
            }
            p.a = from_float<T>(x1);
            p.b = from_float<T>(x2);
            if (rotate) *(Two*)(x + 2 * j) = p;
            if (dst) *(Two*)(dst + 2 * j) = p;
        }
        return;
    }
    for (int j = lane; j < half; j += TL_WAVE) {
        // the two elements that frequency j turns: (j, j + half), or neighbours (2j, 2j + 1) in the
        // pair layout (a projection whose rows were reordered that way at load time)
        const int i1 = pairs ? 2 * j : j, i2 = pairs ? 2 * j + 1 : j + half;
        float x1 = element(i1), x2 = element(i2);
        if (rotate) {
            const float angle = (float)pos * inv_freq[j];
            rope_turn(x1, x2, cosf(angle), sinf(angle));
        }
        if (rotate || parts) {
            x[i1] = from_float<T>(x1);
            x[i2] = from_float<T>(x2);
        }
        if (dst) {
            dst[i1] = from_float<T>(x1);
            dst[i2] = from_float<T>(x2);
        }
    }
}

// The same for bfloat16 rows in the pair layout whose heads are multiples of 8 wide, 16 bytes at a
// time: a work-group owns one token, a thread one 16-byte piece (four pairs of one head) per round.
// Queries are rotated in place, keys rotated and copied to their page in whole pieces, values
// scattered to their transposed place.  (One wave per head, as above, moved 1.7 TB/s on a prompt of
// 2048 tokens; this is for steps of many tokens.)
__global__ __launch_bounds__(256)
void rope_cache_write_rows_kernel(bf16_t* __restrict__ qkv, int row_stride, int q_heads, int kv_heads, int head_dim,
                                  int rot_heads, const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                  const int* __restrict__ token_req, const int* __restrict__ block_table, int bt_stride,
                                  bf16_t* __restrict__ k_plane, bf16_t* __restrict__ v_plane, int page_size) {
    const int t = blockIdx.x;
    const int pos = positions[t];
    const int heads = q_heads + kv_heads + (k_plane ? kv_heads : 0);
    const int pph = head_dim / 8;                                  // pieces per head
    bf16_t* row = qkv + (size_t)t * row_stride;
    size_t page_base = 0;
    if (k_plane) page_base = (size_t)block_table[(size_t)token_req[t] * bt_stride + pos / page_size] * kv_heads * page_size * head_dim;
    const bool stores = k_plane && page_base != 0;                 // page 0 is the sentinel: never written
    const int off = pos % page_size;
    // The token's cosines and sines are worked out once, not once a head: the same 32-bit angle and functions, read
    // back from shared memory by every head's threads (28 query heads and 4 key heads of 128: 2048 tokens 17 -> 12 us).
    __shared__ float2 turn[128];                                   // (head_dim <= 256: the host checks)
    if (inv_freq) {
        for (int j = threadIdx.x; j < head_dim / 2; j += 256) {
            const float angle = (float)pos * inv_freq[j];
            turn[j] = make_float2(cosf(angle), sinf(angle));
        }
        __syncthreads();
    }
    for (int p = threadIdx.x; p < heads * pph; p += 256) {
        const int head = p / pph, d0 = (p % pph) * 8;
        union { uint4 u; uint16_t e[8]; } piece;
        piece.u = *(const uint4*)(row + (size_t)head * head_dim + d0);
        if (head >= q_heads + kv_heads) {                          // value head: [head_dim, page] inside the page
            bf16_t* dst = v_plane + page_base + (size_t)(head - q_heads - kv_heads) * page_size * head_dim + off;
            if (stores) {
#pragma unroll
                for (int e = 0; e < 8; ++e) dst[(size_t)(d0 + e) * page_size].bits = piece.e[e];
            }
            continue;
        }
        const bool rotate = inv_freq && head < rot_heads;
        if (rotate) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bf16_t a, b;
                a.bits = piece.e[2 * j];
                b.bits = piece.e[2 * j + 1];
                float x1 = to_float(a), x2 = to_float(b);
                const float2 cs = turn[d0 / 2 + j];
                rope_turn(x1, x2, cs.x, cs.y);
                piece.e[2 * j] = from_float<bf16_t>(x1).bits;
                piece.e[2 * j + 1] = from_float<bf16_t>(x2).bits;
            }
            *(uint4*)(row + (size_t)head * head_dim + d0) = piece.u;
        }
        if (head >= q_heads && stores)
            *(uint4*)(k_plane + page_base + ((size_t)(head - q_heads) * page_size + off) * head_dim + d0) = piece.u;
    }
}

extern "C" int tl_rope_cache_write(void* qkv, int row_stride, int tokens, int q_heads, int kv_heads,
                                   int head_dim, int rot_heads, const void* positions, const void* inv_freq,
                                   const void* token_req, const void* block_table, int bt_stride,
                                   void* k_plane, void* v_plane, int page_size, int pairs, int act_dtype,
                                   const void* parts, int num_parts, size_t part_stride, int parts_ld,
                                   const void* bias, int bias_f32, hipStream_t stream) {
    TL_REQUIRE(!parts || (num_parts > 0 && parts_ld >= (q_heads + kv_heads + (k_plane ? kv_heads : 0)) * head_dim),
               "rope_cache_write: slabs of partial sums need a count and rows as wide as the heads");
    TL_REQUIRE(tokens >= 0 && q_heads >= 0 && kv_heads >= 0 && head_dim > 0 && head_dim % 2 == 0 && head_dim <= 256,
               "rope_cache_write: bad sizes tokens=%d q_heads=%d kv_heads=%d head_dim=%d (even, at most 256)", tokens, q_heads, kv_heads, head_dim);
    TL_REQUIRE(rot_heads <= q_heads + kv_heads, "rope_cache_write: rot_heads %d exceeds q+k heads", rot_heads);
    TL_REQUIRE((k_plane == nullptr) == (v_plane == nullptr), "rope_cache_write: give both planes or none");
    TL_REQUIRE(!k_plane || (block_table && token_req && page_size > 0 && bt_stride > 0),
               "rope_cache_write: cache write needs block table, token_req and page size");
    TL_REQUIRE(row_stride >= (q_heads + (k_plane ? 2 * kv_heads : kv_heads)) * head_dim,
               "rope_cache_write: row stride %d too small", row_stride);
    if (tokens == 0) return TL_OK;
    const int heads = q_heads + kv_heads + (k_plane ? kv_heads : 0);
    // pairs as one access: rows and planes start on a multiple of two elements (eight bytes covers both dtypes)
    const int pair_aligned = row_stride % 2 == 0 && ((uintptr_t)qkv % 8) == 0 && ((uintptr_t)k_plane % 8) == 0;
    if (act_dtype == TL_DT_BF16 && pairs && !parts && tokens >= 64 && head_dim % 8 == 0 && row_stride % 8 == 0 &&
        ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)k_plane % 16) == 0 && (!inv_freq || ((uintptr_t)inv_freq % 16) == 0)) {
        rope_cache_write_rows_kernel<<<dim3(tokens), dim3(256), 0, stream>>>((bf16_t*)qkv, row_stride, q_heads, kv_heads, head_dim, rot_heads,
            (const int*)positions, (const float*)inv_freq, (const int*)token_req, (const int*)block_table, bt_stride,
            (bf16_t*)k_plane, (bf16_t*)v_plane, page_size);
        TL_CHECK_LAUNCH("rope_cache_write");
        return TL_OK;
    }
    dim3 grid(tokens, (heads + ROPE_HEADS_PER_GROUP - 1) / ROPE_HEADS_PER_GROUP), block(ROPE_HEADS_PER_GROUP * TL_WAVE);
    if (act_dtype == TL_DT_F32)
        rope_cache_write_kernel<float><<<grid, block, 0, stream>>>((float*)qkv, row_stride, q_heads, kv_heads, head_dim, rot_heads,
            (const int*)positions, (const float*)inv_freq, (const int*)token_req, (const int*)block_table, bt_stride,
            (float*)k_plane, (float*)v_plane, page_size, pairs, pair_aligned, (const float*)parts, num_parts, part_stride, parts_ld, bias, bias_f32);
    else if (act_dtype == TL_DT_BF16)
        rope_cache_write_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)qkv, row_stride, q_heads, kv_heads, head_dim, rot_heads,
            (const int*)positions, (const float*)inv_freq, (const int*)token_req, (const int*)block_table, bt_stride,
            (bf16_t*)k_plane, (bf16_t*)v_plane, page_size, pairs, pair_aligned, (const float*)parts, num_parts, part_stride, parts_ld, bias, bias_f32);
    else TL_REQUIRE(false, "rope_cache_write: unknown dtype %d", act_dtype);
    TL_CHECK_LAUNCH("rope_cache_write");
    return TL_OK;
}

// ------------------------------------------------------------------ SwiGLU gate
// out[t, i] = silu(gu[t, i]) * gu[t, inter + i], silu(g) = g / (1 + exp(-g)).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, size_t total) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / inter;
    const int i = (int)(idx % inter);
    const float g = to_float(gu[t * 2 * inter + i]);
    const float u = to_float(gu[t * 2 * inter + inter + i]);
    out[idx] = from_float<T>(g / (1.f + expf(-g)) * u);
}

extern "C" int tl_swiglu(const void* gu, void* out, int tokens, int inter, int act_dtype, hipStream_t stream) {
    TL_REQUIRE(tokens >= 0 && inter > 0, "swiglu: bad sizes tokens=%d inter=%d", tokens, inter);
    const size_t total = (size_t)tokens * inter;
    if (total == 0) return TL_OK;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    if (act_dtype == TL_DT_F32)
        swiglu_kernel<float><<<grid, block, 0, stream>>>((const float*)gu, (float*)out, inter, total);
    else if (act_dtype == TL_DT_BF16)
        swiglu_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, inter, total);
    else TL_REQUIRE(false, "swiglu: unknown dtype %d", act_dtype);
    TL_CHECK_LAUNCH("swiglu");
    return TL_OK;
}

// ------------------------------------------------------------------ streaming read (a yardstick)
// Reads `bytes` of memory once, as fast as the machine lets a kernel read: every work-group walks a
// contiguous share in 16-byte pieces, eight requests per thread on their way, and folds what it read into one
// word per work-group (written to `sink`, so that no read can be dropped).  What it measures is the rate at
// which this GPU delivers memory to any kernel that only reads; the benchmark quotes the decode step against it.
#define STREAM_THREADS 256
#define STREAM_DEPTH 8
__global__ __launch_bounds__(STREAM_THREADS) void stream_read_kernel(const uint4* __restrict__ p, size_t pieces,
                                                                     size_t per_group, uint32_t* __restrict__ sink) {
    const size_t begin = (size_t)blockIdx.x * per_group;
    const size_t end = begin + per_group < pieces ? begin + per_group : pieces;
    uint32_t acc = 0;
    size_t i = begin + threadIdx.x;
    for (; i + (STREAM_DEPTH - 1) * STREAM_THREADS < end; i += STREAM_DEPTH * STREAM_THREADS) {
        uint4 v[STREAM_DEPTH];
#pragma unroll
        for (int u = 0; u < STREAM_DEPTH; ++u) v[u] = p[i + (size_t)u * STREAM_THREADS];
#pragma unroll
        for (int u = 0; u < STREAM_DEPTH; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < end; i += STREAM_THREADS) {
        const uint4 v = p[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
#pragma unroll
    for (int o = TL_WAVE / 2; o > 0; o >>= 1) acc ^= __shfl_xor(acc, o, TL_WAVE);
    __shared__ uint32_t part[STREAM_THREADS / TL_WAVE];
    if (threadIdx.x % TL_WAVE == 0) part[threadIdx.x / TL_WAVE] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t all = 0;
        for (int w = 0; w < STREAM_THREADS / TL_WAVE; ++w) all ^= part[w];
        sink[blockIdx.x] = all;
    }
}

// Work-groups the read is dealt to by default (`sink` needs one 32-bit word per work-group).
extern "C" int tl_stream_read_groups() { return 8192; }     // measured: 256 give 5.6 TB/s, 2048 6.2, 8192 6.3, 16384 6.2

extern "C" int tl_stream_read(const void* data, size_t bytes, void* sink, int groups, hipStream_t stream) {
    TL_REQUIRE(data != nullptr && sink != nullptr && bytes >= 16 && ((uintptr_t)data % 16) == 0,
               "stream_read: needs 16-byte aligned memory of at least 16 bytes and a sink");
    TL_REQUIRE(groups >= 0 && groups <= 65536, "stream_read: %d work-groups", groups);
    const size_t pieces = bytes / 16;
    if (groups == 0) groups = tl_stream_read_groups();
    const size_t per_group = (pieces + groups - 1) / groups;
    stream_read_kernel<<<dim3(groups), dim3(STREAM_THREADS), 0, stream>>>((const uint4*)data, pieces, per_group, (uint32_t*)sink);
    TL_CHECK_LAUNCH("stream_read");
    return TL_OK;
}
