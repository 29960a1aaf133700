// Paged grouped-query attention over the tokens of one step, general kernel.
//
// One kernel serves prompt portions and decode tokens alike.  A work-group owns a
// "tile" of up to 16 rows that share one KV head: `tq` consecutive new tokens of one
// request times the `gcap` query heads of the group (tq * gcap <= 16), so keys and
// values are read once for the whole group.  The keys of a request lie in pages of
// `page` tokens found through its block-table row; a row at position p sees the keys
// max(0, p - window + 1) .. p (window == 0: from 0).  Scores, running maximum, sum and
// the accumulator are float; the softmax is computed online, tile of keys by tile of
// keys, with key tiles aligned to absolute positions.  With splits > 1 the range of
// key tiles is divided over blockIdx.z and a second kernel merges the parts.
//
// Keys lie in their pages as [kv_head][position][d]; values lie transposed,
// [kv_head][d][position], which is the layout the matrix-core kernel below reads directly.
//
// Compiled per head size: -DTL_HEAD_DIM=<multiple of 16>.  A library serves the head sizes
// TL_HEAD_DIM - 14 .. TL_HEAD_DIM (even ones): the general kernel takes the true size `hd` at run time and
// treats the dimensions from hd up to TL_HEAD_DIM as zeros that are neither read nor written; the
// matrix-core kernels are for hd == TL_HEAD_DIM.
#include "common.h"
#include <type_traits>

#ifndef TL_HEAD_DIM
#error "compile with -DTL_HEAD_DIM=<head size>"
#endif
static_assert(TL_HEAD_DIM % 16 == 0 && TL_HEAD_DIM >= 16 && TL_HEAD_DIM <= 256, "head size: multiple of 16 up to 256");

#define AT_ROWS 16
#define AT_HD TL_HEAD_DIM
#define AT_KT (AT_HD <= 128 ? 32 : 16)                        // keys per tile
#define AT_DPT (AT_HD / 16)                                   // output dims per thread

struct AttnArgs {
    const void* q;            // [tokens, q_stride], head h at column h * HD
    void* out;                // [tokens, heads * HD]
    const void* k_plane;      // [pages, kv_heads, page, HD]
    const void* v_plane;      // [pages, kv_heads, HD, page]: values lie transposed inside a page
    const int* block_table;   // [requests, bt_stride]
    const int* req_indptr;    // [requests + 1] first new token of each request
    const int* ctx_lens;      // [requests] tokens cached before this step
    const int* tile_req;      // [tiles]
    const int* tile_tok0;     // [tiles] first new token of the tile, relative to its request
    float* part_o;            // [tokens * heads, splits, HD] (splits > 1)
    float* part_ml;           // [tokens * heads, splits, 2]
    int q_stride, bt_stride, heads, kv_heads, page, window, tq, gcap, splits;
    int hd;                   // the true head size, <= HD: width of a head in q, out and the planes
    int page_shift;           // log2(page) when page is a power of two, else -1
    int units;                // compute units of the GPU (the prompt kernel's order of work)
    float scale;
};

// key position -> (logical block, offset in its page); a shift and a mask for the usual
// power-of-two pages (an integer division by a run-time page size costs ~25 instructions)
__device__ __forceinline__ void split_key(int key, int page, int shift, int& blk, int& off) {
    if (shift >= 0) {
        blk = key >> shift;
        off = key & (page - 1);
    } else {
        blk = key / page;
        off = key - blk * page;
    }
}

// Four bfloat16 values of the keys key0 .. key0 + 3 with those at or beyond key_hi set to zero.
// A page may hold anything where no key has been written yet (another request's leftovers, even
// Inf or NaN); a probability of zero does not stop those from reaching the sum, a zero value does.
__device__ __forceinline__ uint2 keep_written(uint2 v, int key0, int key_hi) {
    const int n = key_hi - key0;                  // written keys among the four
    if (n >= 4) return v;
    if (n <= 0) return make_uint2(0, 0);
    if (n == 1) return make_uint2(v.x & 0xffffu, 0);
    if (n == 2) return make_uint2(v.x, 0);
    return make_uint2(v.x, v.y & 0xffffu);
}

template <typename T>
__global__ __launch_bounds__(256) void paged_attention_kernel(AttnArgs a) {
    __shared__ float qs[AT_ROWS][AT_HD + 1];
    __shared__ float ks[AT_KT][AT_HD + 1];
    __shared__ float vs[AT_KT][AT_HD + 1];
    __shared__ float ps[AT_ROWS][AT_KT + 1];

    const int tile = blockIdx.x;
    const int group = a.heads / a.kv_heads;
    const int chunks = (group + a.gcap - 1) / a.gcap;       // head chunks per KV head
    const int kvh = blockIdx.y / chunks;
    const int g0 = (blockIdx.y % chunks) * a.gcap;           // first head of this chunk inside the group
    const int gcount = min(a.gcap, group - g0);
    const int split = blockIdx.z;

    // without a tile list (a step in which every request decodes one token): tile i is the token of request i
    const bool one_each = a.tile_req == nullptr;
    const int req = one_each ? tile : a.tile_req[tile];
    const int tok0 = one_each ? 0 : a.tile_tok0[tile];
    const int first = one_each ? req : a.req_indptr[req];
    const int n_new = one_each ? 1 : a.req_indptr[req + 1] - first;
    const int ctx = a.ctx_lens[req];
    const int ntok = min(a.tq, n_new - tok0);                // tokens of this tile

    const int tid = threadIdx.x;
    const int row = tid / 16;                                 // 0..15: my row in scores and output
    const int sub = tid % 16;
    const int r_tok = row / a.gcap, r_g = row % a.gcap;
    const bool row_ok = r_tok < ntok && r_g < gcount;
    const int r_pos = ctx + tok0 + r_tok;                     // position of my row's query
    const int r_head = kvh * group + g0 + r_g;
    const int r_token = first + tok0 + r_tok;                 // flat token index

    // queries -> shared, as float
    const T* q = (const T*)a.q;
    for (int i = tid; i < AT_ROWS * AT_HD; i += 256) {
        const int rr = i / AT_HD, d = i % AT_HD;
        const int tt = rr / a.gcap, gg = rr % a.gcap;
        float v = 0.f;
        if (tt < ntok && gg < gcount && d < a.hd)
            v = to_float(q[(size_t)(first + tok0 + tt) * a.q_stride + (size_t)(kvh * group + g0 + gg) * a.hd + d]);
        qs[rr][d] = v;
    }

    // range of keys of the tile, in key tiles aligned to absolute positions
    const int key_hi = ctx + tok0 + ntok;                      // exclusive
    const int key_lo = a.window > 0 ? max(0, ctx + tok0 - a.window + 1) : 0;
    const int kt_first = key_lo / AT_KT;
    const int kt_last = (key_hi + AT_KT - 1) / AT_KT;          // exclusive
    const int per_split = (kt_last - kt_first + a.splits - 1) / a.splits;
    const int kt_begin = kt_first + split * per_split;
    const int kt_end = min(kt_last, kt_begin + per_split);

    const T* kp = (const T*)a.k_plane;
    const T* vp = (const T*)a.v_plane;
    const int* bt = a.block_table + (size_t)req * a.bt_stride;

    float m = -INFINITY, l = 0.f;
    float acc[AT_DPT];
#pragma unroll
    for (int i = 0; i < AT_DPT; ++i) acc[i] = 0.f;

    for (int kt = kt_begin; kt < kt_end; ++kt) {
        const int kbase = kt * AT_KT;
        __syncthreads();   // previous tile fully consumed (and qs written, first time)
        for (int i = tid; i < AT_KT * AT_HD; i += 256) {
            const int j = i / AT_HD, d = i % AT_HD;
            const int pos = kbase + j;
            float kv = 0.f, vv = 0.f;
            if (pos < key_hi && d < a.hd) {
                const int pg = bt[pos / a.page];
                const size_t head = ((size_t)pg * a.kv_heads + kvh) * a.page * a.hd;
                kv = to_float(kp[head + (size_t)(pos % a.page) * a.hd + d]);
                vv = to_float(vp[head + (size_t)d * a.page + (pos % a.page)]);
            }
            ks[j][d] = kv;
            vs[j][d] = vv;
        }
        __syncthreads();

        // scores of my row against keys sub, sub + 16, ...
        float s[AT_KT / 16 > 0 ? AT_KT / 16 : 1];
        float tmax = -INFINITY;
#pragma unroll
        for (int c = 0; c < (AT_KT + 15) / 16; ++c) {
            const int j = sub + 16 * c;
            float dot = -INFINITY;
            if (j < AT_KT) {
                const int pos = kbase + j;
                const bool seen = row_ok && pos <= r_pos && pos < key_hi && (a.window <= 0 || pos > r_pos - a.window);
                if (seen) {
                    float d0 = 0.f;
#pragma unroll 8
                    for (int d = 0; d < AT_HD; ++d) d0 = fmaf(qs[row][d], ks[j][d], d0);
                    dot = d0 * a.scale;
                }
            }
            s[c] = dot;
            tmax = fmaxf(tmax, dot);
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, o, TL_WAVE));
        const float m_new = fmaxf(m, tmax);
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        float psum = 0.f;
#pragma unroll
        for (int c = 0; c < (AT_KT + 15) / 16; ++c) {
            const int j = sub + 16 * c;
            if (j < AT_KT) {
                const float p = (s[c] == -INFINITY) ? 0.f : expf(s[c] - m_new);
                ps[row][j] = p;
                psum += p;
            }
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, TL_WAVE);
        l = l * alpha + psum;
        m = m_new;
        __syncthreads();   // ps complete
#pragma unroll
        for (int i = 0; i < AT_DPT; ++i) acc[i] *= alpha;
        for (int j = 0; j < AT_KT; ++j) {
            const float p = ps[row][j];
#pragma unroll
            for (int i = 0; i < AT_DPT; ++i) acc[i] = fmaf(p, vs[j][sub + 16 * i], acc[i]);
        }
    }

    if (!row_ok) return;
    if (a.splits == 1) {
        T* o = (T*)a.out + (size_t)r_token * a.heads * a.hd + (size_t)r_head * a.hd;
        const float inv = 1.f / l;
#pragma unroll
        for (int i = 0; i < AT_DPT; ++i)
            if (sub + 16 * i < a.hd) o[sub + 16 * i] = from_float<T>(acc[i] * inv);
    } else {
        const size_t pr = ((size_t)r_token * a.heads + r_head) * a.splits + split;
        float* o = a.part_o + pr * AT_HD;
#pragma unroll
        for (int i = 0; i < AT_DPT; ++i) o[sub + 16 * i] = acc[i];
        if (sub == 0) {
            a.part_ml[pr * 2] = m;
            a.part_ml[pr * 2 + 1] = l;
        }
    }
}


// =====================================================================================
// The same attention on the matrix cores, for bfloat16 (pages of a multiple of 4 tokens).
//
// A wave owns the tile's 16 rows and walks the keys in chunks of 32.  Both products run
// transposed so that no operand ever changes layout between them:
//   S^T[key, row] = K[key, :] . Q[row, :]      A = 16 keys of K (rows of a page, d contiguous),
//                                              B = Q;  a lane ends up with the scores of its
//                                              row (lane % 16) for the keys 4g .. 4g+3 of each
//                                              16-key half, g = lane / 16;
//   O^T[d, row]   = V^T[d, key] . P^T[key, row] A = V^T, read straight from the transposed value
//                                              pages as two 8-byte pieces (4 keys of each half),
//                                              B = the lane's own eight probabilities.
// The k-slots of the second product are dealt to keys as {4g..4g+3 of the first half,
// 4g..4g+3 of the second}, for A and B alike, which is why no shuffle or shared memory is
// needed.  The online softmax works in base 2 on scores pre-multiplied by scale * log2(e);
// running maximum and sum are float, probabilities are rounded to bfloat16 for the product
// with V.  The waves of a work-group (NW: four or eight) take the chunks of the tile's key range (or of its
// split) in turn and merge their states pairwise through shared memory at the end.  Eight waves with half as
// many parts per request are as many waves on as many keys, with half the partial results to write, read and
// merge, or none (7B sizes, contexts of 2048: the decode step at batch 1 / 8 / 64 3.33 / 3.72 / 5.34 ->
// 3.28 / 3.66 / 5.24 ms); where every request has a work-group of four to itself and the compute units are
// full with those, four stay ahead (batch 128: 7.61 against 7.75 ms).
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

union FragK {
    uint4 u;
    uint2 h[2];
    bf16x8_t v;
    uint16_t e[8];
};

#define ATM_DC ((AT_HD + 31) / 32)
#define ATM_DT (AT_HD / 16)
#define ATM_SLOT (ATM_DT * 256 + 128)      // floats one wave parks in shared memory
#define ATM_BT_MAX 2048                    // block-table entries a work-group keeps in shared memory

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
// The larger of a lane's value and that of lane ^ 32 (lane ^ 16): the halves (the rows of 16 lanes) change places in
// the vector unit, where a shuffle would go through shared memory and the step would wait for the trip.
__device__ __forceinline__ float max_across_halves(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float max_across_rows(float x) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

template <int NW>
__global__ __launch_bounds__(64 * NW) void paged_attention_mfma_kernel(AttnArgs a) {
    __shared__ float park[(NW / 2) * ATM_SLOT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, g = lane >> 4;

    const int tile = blockIdx.x;
    const int group = a.heads / a.kv_heads;
    const int chunks_h = (group + a.gcap - 1) / a.gcap;
    const int kvh = blockIdx.y / chunks_h;
    const int g0 = (blockIdx.y % chunks_h) * a.gcap;
    const int gcount = min(a.gcap, group - g0);
    const int split = blockIdx.z;

    // Without a tile list (a step in which every request decodes one token) tile i is the token of request
    // i: nothing has to be looked up before the request's length, its block table and the query are
    // requested, all three at once; with a list each of these waits for the one before it.
    const bool one_each = a.tile_req == nullptr;
    const int req = one_each ? tile : a.tile_req[tile];
    __shared__ int bt_s[ATM_BT_MAX];
    const int* bt_g = a.block_table + (size_t)req * a.bt_stride;
    const bool bt_whole = a.bt_stride <= ATM_BT_MAX;        // the whole row, before the length says which part is needed
    if (bt_whole)
        for (int i = threadIdx.x; i < a.bt_stride; i += 64 * NW) bt_s[i] = bt_g[i];
    const int tok0 = one_each ? 0 : a.tile_tok0[tile];
    const int first = one_each ? req : a.req_indptr[req];
    const int n_new = one_each ? 1 : a.req_indptr[req + 1] - first;
    const int ctx = a.ctx_lens[req];
    const int ntok = min(a.tq, n_new - tok0);

    const int r_tok = li / a.gcap, r_g = li % a.gcap;
    const bool row_ok = r_tok < ntok && r_g < gcount;
    const int r_pos = ctx + tok0 + r_tok;
    const int r_lo = a.window > 0 ? r_pos - a.window + 1 : 0;
    const int r_head = kvh * group + g0 + r_g;
    const int r_token = first + tok0 + r_tok;

    // my row's query, as B operand of the first product: d = 32 c + 8 g .. + 8
    FragK qf[ATM_DC];
    {
        const bf16_t* q = (const bf16_t*)a.q + (size_t)r_token * a.q_stride + (size_t)r_head * AT_HD;
#pragma unroll
        for (int c = 0; c < ATM_DC; ++c) {
            const int d = 32 * c + 8 * g;
            qf[c].u = (row_ok && d + 8 <= AT_HD) ? *(const uint4*)(q + d) : make_uint4(0, 0, 0, 0);
        }
    }

    const int key_hi = ctx + tok0 + ntok;
    const int key_lo = a.window > 0 ? max(0, ctx + tok0 - a.window + 1) : 0;
    const int ch_first = key_lo / 32;
    const int ch_last = (key_hi + 31) / 32;
    const int per_split = (ch_last - ch_first + a.splits - 1) / a.splits;
    const int ch_begin = ch_first + split * per_split;
    const int ch_end = min(ch_last, ch_begin + per_split);

    const bf16_t* kp = (const bf16_t*)a.k_plane;
    const bf16_t* vp = (const bf16_t*)a.v_plane;
    const int page = a.page;
    // The block-table entries of the keys this work-group reads go to shared memory first: a
    // page lookup in the loop is then a shared-memory read instead of a memory access that the
    // key and value loads would have to wait for (two memory latencies in a row per chunk).
    const int blk0 = bt_whole ? 0 : (ch_begin * 32) / page;
    const int blk_n = ch_begin < ch_end ? (min(ch_end * 32, key_hi) - 1) / page - blk0 + 1 : 0;
    const bool bt_local = bt_whole || blk_n <= ATM_BT_MAX;
    if (bt_local) {
        if (!bt_whole)
            for (int i = threadIdx.x; i < blk_n; i += 64 * NW) bt_s[i] = bt_g[blk0 + i];
        __syncthreads();
    }
#define ATM_PAGE_OF(blk) (bt_local ? bt_s[(blk) - blk0] : bt_g[(blk)])
    const float scale2 = a.scale * 1.44269504088896341f;
    // smallest query position and largest window start over the rows of the tile (uniform)
    const int tile_pos_min = ctx + tok0;
    const int tile_lo_max = a.window > 0 ? max(0, ctx + tok0 + ntok - 1 - a.window + 1) : 0;

    float m = -INFINITY, l = 0.f;
    f32x4_t acc[ATM_DT];
#pragma unroll
    for (int t = 0; t < ATM_DT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Keys and values of a chunk are fetched together: the value loads do not wait for the
    // scores.  (Fetching the next chunk ahead as well doubles the registers, halves the waves
    // per SIMD and measured slower for decode and prompt steps alike.)
    FragK kf[2][ATM_DC];
    uint2 vfa[ATM_DT], vfb[ATM_DT];
#define ATM_FETCH(KF, VA, VB, chunk)                                                                         \
    {                                                                                                        \
        const int kb_ = (chunk) * 32;                                                                        \
        _Pragma("unroll") for (int hf = 0; hf < 2; ++hf) {                                                   \
            int blk, off;                                                                                    \
            split_key(min(kb_ + 16 * hf + li, key_hi - 1), page, a.page_shift, blk, off);                    \
            const bf16_t* krow = kp + ((size_t)ATM_PAGE_OF(blk) * kv_stride + kvh_off + off * AT_HD);        \
            _Pragma("unroll") for (int c = 0; c < ATM_DC; ++c) {                                             \
                const int d = 32 * c + 8 * g;                                                                \
                KF[hf][c].u = (d + 8 <= AT_HD) ? *(const uint4*)(krow + d) : make_uint4(0, 0, 0, 0);         \
            }                                                                                                \
        }                                                                                                    \
        const int ka = kb_ + 4 * g, kb = kb_ + 16 + 4 * g;                                                   \
        const bool oka = ka < key_hi, okb = kb < key_hi;                                                     \
        int blka, offa, blkb, offb;                                                                          \
        split_key(ka, page, a.page_shift, blka, offa);                                                       \
        split_key(kb, page, a.page_shift, blkb, offb);                                                       \
        const bf16_t* va = vp + ((size_t)(oka ? ATM_PAGE_OF(blka) : 0) * kv_stride + kvh_off + offa + li * page); \
        const bf16_t* vb = vp + ((size_t)(okb ? ATM_PAGE_OF(blkb) : 0) * kv_stride + kvh_off + offb + li * page); \
        _Pragma("unroll") for (int t = 0; t < ATM_DT; ++t) {                                                 \
            VA[t] = oka ? *(const uint2*)(va + 16 * t * page) : make_uint2(0, 0);                            \
            VB[t] = okb ? *(const uint2*)(vb + 16 * t * page) : make_uint2(0, 0);                            \
        }                                                                                                    \
        if (kb_ + 32 > key_hi) {          /* the last chunk: keys that are not written yet */                 \
            _Pragma("unroll") for (int t = 0; t < ATM_DT; ++t) {                                             \
                VA[t] = keep_written(VA[t], ka, key_hi);                                                     \
                VB[t] = keep_written(VB[t], kb, key_hi);                                                     \
            }                                                                                                \
        }                                                                                                    \
    }

    const size_t kv_stride = (size_t)a.kv_heads * page * AT_HD;     /* elements per page, all KV heads */
    const int kvh_off = kvh * page * AT_HD;

    int ch = ch_begin + wave;
    if (ch < ch_end) ATM_FETCH(kf, vfa, vfb, ch)
    for (; ch < ch_end; ch += NW) {
        const int kbase = ch * 32;
        // ---- scores: two halves of 16 keys
        f32x4_t sc[2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            f32x4_t sacc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < ATM_DC; ++c)
                sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[hf][c].v, qf[c].v, sacc, 0, 0, 0);
            sc[hf] = sacc;
        }
        // ---- mask, running maximum, probabilities
        // A chunk that every row of the tile sees whole (all but those on the diagonal, at a
        // window's edge or at the end of the keys) needs no mask: the branch is uniform.
        float s[8];
        float mloc = -INFINITY;
        if (kbase + 31 <= tile_pos_min && kbase >= tile_lo_max) {
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float x = sc[hf][v] * scale2;
                    s[4 * hf + v] = x;
                    mloc = fmaxf(mloc, x);
                }
        } else {
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = kbase + 16 * hf + 4 * g + v;
                    const bool seen = row_ok && key <= r_pos && key >= r_lo;
                    const float x = seen ? sc[hf][v] * scale2 : -INFINITY;
                    s[4 * hf + v] = x;
                    mloc = fmaxf(mloc, x);
                }
        }
        mloc = max_across_halves(max_across_rows(mloc));
        const float m_new = fmaxf(m, mloc);
        const float alpha = (m == -INFINITY) ? 0.f : fast_exp2(m - m_new);
        FragK pf;
        float psum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float p = (s[i] == -INFINITY) ? 0.f : fast_exp2(s[i] - m_new);
            psum += p;
            pf.v[i] = (__bf16)p;
        }
        l = l * alpha + psum;
        // ---- values: O^T += V^T . P^T; the accumulators are rescaled only when some row's maximum moved
        const bool moved = __any(m_new != m);
        m = m_new;
#pragma unroll
        for (int t = 0; t < ATM_DT; ++t) {
            FragK vf;
            vf.h[0] = vfa[t];
            vf.h[1] = vfb[t];
            if (moved) acc[t] *= alpha;
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, acc[t], 0, 0, 0);
        }
        if (ch + NW < ch_end) ATM_FETCH(kf, vfa, vfb, ch + NW)
    }
#undef ATM_FETCH
#undef ATM_PAGE_OF

    // ---- merge the waves: the upper half of those left hands its state to the lower half, until one is left
#pragma unroll
    for (int half = NW / 2; half >= 1; half >>= 1) {
        __syncthreads();
        if (wave >= half && wave < 2 * half) {
            float* dst = park + (size_t)(wave - half) * ATM_SLOT;
#pragma unroll
            for (int t = 0; t < ATM_DT; ++t) *(f32x4_t*)(dst + (t * 64 + lane) * 4) = acc[t];
            dst[ATM_DT * 256 + lane] = m;
            dst[ATM_DT * 256 + 64 + lane] = l;
        }
        __syncthreads();
        if (wave < half) {
            const float* src = park + (size_t)wave * ATM_SLOT;
            const float mo = src[ATM_DT * 256 + lane], lo = src[ATM_DT * 256 + 64 + lane];
            const float mm = fmaxf(m, mo);
            const float sa = (m == -INFINITY) ? 0.f : fast_exp2(m - mm);
            const float sb = (mo == -INFINITY) ? 0.f : fast_exp2(mo - mm);
#pragma unroll
            for (int t = 0; t < ATM_DT; ++t) acc[t] = acc[t] * sa + *(const f32x4_t*)(src + (t * 64 + lane) * 4) * sb;
            l = l * sa + lo * sb;
            m = mm;
        }
    }
    if (wave != 0) return;
    l += __shfl_xor(l, 16, TL_WAVE);
    l += __shfl_xor(l, 32, TL_WAVE);
    if (!row_ok) return;
    if (a.splits == 1) {
        bf16_t* o = (bf16_t*)a.out + (size_t)r_token * a.heads * AT_HD + (size_t)r_head * AT_HD;
        const float inv = 1.f / l;
#pragma unroll
        for (int t = 0; t < ATM_DT; ++t) {
            union { uint2 u; uint16_t e[4]; } pk;
#pragma unroll
            for (int v = 0; v < 4; ++v) pk.e[v] = from_float<bf16_t>(acc[t][v] * inv).bits;
            *(uint2*)(o + 16 * t + 4 * g) = pk.u;
        }
    } else {
        const size_t pr = ((size_t)r_token * a.heads + r_head) * a.splits + split;
        float* o = a.part_o + pr * AT_HD;
#pragma unroll
        for (int t = 0; t < ATM_DT; ++t) *(f32x4_t*)(o + 16 * t + 4 * g) = acc[t];
        if (g == 0) {
            a.part_ml[pr * 2] = m * 0.69314718055994531f;      // back to natural logarithms for the merge
            a.part_ml[pr * 2 + 1] = l;
        }
    }
}

// =====================================================================================
// Prompt portions on the matrix cores: 64 rows per work-group, keys and values through
// shared memory.
//
// The kernel above lets every wave fetch its own keys, which is right when the waves of a
// work-group split the keys of one 16-row tile among themselves (decode).  For a prompt
// portion there are many row tiles over the same keys: here the four waves of a work-group
// each own one 16-row tile (64 rows: consecutive tokens x the heads of one KV group), fetch
// every 32-key chunk once, together, into shared memory (two buffers; the next chunk is on
// its way from memory while the current one is multiplied), and read their operands from
// there.  The arithmetic per wave is the same as above (transposed products, base-2 online
// softmax in float).  A wave skips the chunks that lie beyond all of its rows.
// Built for head sizes up to 128.
#if AT_HD <= 128
#define ATP_KROW (AT_HD + 8)          // bfloat16 elements between key rows in shared memory
#define ATP_VROW 36                   // between value rows (32 keys + 4 of padding)
#define ATP_KPIECES (32 * AT_HD / 8)  // 16-byte pieces of a key chunk
#define ATP_VPIECES (AT_HD * 8)       // 8-byte pieces (4 keys of one d) of a value chunk
#define ATP_KPT ((ATP_KPIECES + 255) / 256)
#define ATP_VPT ((ATP_VPIECES + 255) / 256)

__global__ __launch_bounds__(256) void paged_attention_prefill_kernel(AttnArgs a) {
    __shared__ __attribute__((aligned(16))) bf16_t ks[2][32 * ATP_KROW];
    __shared__ __attribute__((aligned(16))) bf16_t vs[2][AT_HD * ATP_VROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, g = lane >> 4;

    // later tiles of a prompt see more keys: start them first, each with all its key/value heads (launch
    // order runs along x first), so that the short ones fill the end
    const int rank = blockIdx.y * gridDim.x + blockIdx.x;
    const int tile = gridDim.x - 1 - rank / (int)gridDim.y;
    const int by = rank % (int)gridDim.y;
    const int group = a.heads / a.kv_heads;
    const int chunks_h = (group + a.gcap - 1) / a.gcap;
    const int kvh = by / chunks_h;
    const int g0 = (by % chunks_h) * a.gcap;
    const int gcount = min(a.gcap, group - g0);

    const int req = a.tile_req[tile];
    const int tok0 = a.tile_tok0[tile];
    const int first = a.req_indptr[req];
    const int n_new = a.req_indptr[req + 1] - first;
    const int ctx = a.ctx_lens[req];
    const int ntok = min(a.tq, n_new - tok0);           // a.tq: tokens of a 64-row tile

    const int row = wave * 16 + li;                      // my row among the 64
    const int r_tok = row / a.gcap, r_g = row % a.gcap;
    const bool row_ok = r_tok < ntok && r_g < gcount;
    const int r_pos = ctx + tok0 + r_tok;
    const int r_lo = a.window > 0 ? r_pos - a.window + 1 : 0;
    const int r_head = kvh * group + g0 + r_g;
    const int r_token = first + tok0 + r_tok;
    // positions of my wave's rows (uniform per wave)
    const int w_tok_lo = min((wave * 16) / a.gcap, ntok - 1), w_tok_hi = min((wave * 16 + 15) / a.gcap, ntok - 1);
    const int w_pos_min = ctx + tok0 + w_tok_lo, w_pos_max = ctx + tok0 + w_tok_hi;
    const int w_lo_max = a.window > 0 ? max(0, w_pos_max - a.window + 1) : 0;
    const int w_lo_min = a.window > 0 ? max(0, w_pos_min - a.window + 1) : 0;
    const bool wave_has_rows = (wave * 16) / a.gcap < ntok;

    FragK qf[ATM_DC];
    {
        const bf16_t* q = (const bf16_t*)a.q + (size_t)r_token * a.q_stride + (size_t)r_head * AT_HD;
#pragma unroll
        for (int c = 0; c < ATM_DC; ++c) {
            const int d = 32 * c + 8 * g;
            qf[c].u = (row_ok && d + 8 <= AT_HD) ? *(const uint4*)(q + d) : make_uint4(0, 0, 0, 0);
        }
    }

    const int key_hi = ctx + tok0 + ntok;
    const int key_lo = a.window > 0 ? max(0, ctx + tok0 - a.window + 1) : 0;
    const int ch_begin = key_lo / 32, ch_end = (key_hi + 31) / 32;

    const bf16_t* kp = (const bf16_t*)a.k_plane;
    const bf16_t* vp = (const bf16_t*)a.v_plane;
    const int page = a.page;
    const float scale2 = a.scale * 1.44269504088896341f;
    // block-table entries of the tile's keys, in shared memory (see the kernel above)
    __shared__ int bt_s[ATM_BT_MAX];
    const int* bt_g = a.block_table + (size_t)req * a.bt_stride;
    const int blk0 = (ch_begin * 32) / page;
    const int blk_n = ch_begin < ch_end ? (key_hi - 1) / page - blk0 + 1 : 0;
    const bool bt_local = blk_n <= ATM_BT_MAX;
    if (bt_local) {
        for (int i = tid; i < blk_n; i += 256) bt_s[i] = bt_g[blk0 + i];
        __syncthreads();
    }
#define ATP_PAGE_OF(blk) (bt_local ? bt_s[(blk) - blk0] : bt_g[(blk)])

    // two register stages: chunk c+1 (fetched during the previous iteration) and chunk c+2
    uint4 kst[ATP_KPT], kst2[ATP_KPT];
    uint2 vst[ATP_VPT], vst2[ATP_VPT];
    // which pieces of a chunk this thread fetches does not change from chunk to chunk
    int kj[ATP_KPT], kpc[ATP_KPT], vd[ATP_VPT], vq[ATP_VPT];
#pragma unroll
    for (int i = 0; i < ATP_KPT; ++i) { const int idx = tid + 256 * i; kj[i] = idx / (AT_HD / 8); kpc[i] = (idx % (AT_HD / 8)) * 8; }
#pragma unroll
    for (int i = 0; i < ATP_VPT; ++i) { const int idx = tid + 256 * i; vd[i] = idx / 8; vq[i] = (idx % 8) * 4; }
    const size_t kv_stride = (size_t)a.kv_heads * page * AT_HD;     // elements per page, all KV heads
    const int kvh_off = kvh * page * AT_HD;
#define ATP_FETCH(KS_, VS_, chunk)                                                                         \
    {                                                                                                      \
        const int kb_ = (chunk) * 32;                                                                      \
        _Pragma("unroll") for (int i = 0; i < ATP_KPT; ++i) {                                              \
            KS_[i] = make_uint4(0, 0, 0, 0);                                                               \
            if (tid + 256 * i < ATP_KPIECES) {                                                             \
                int blk, off;                                                                              \
                split_key(min(kb_ + kj[i], key_hi - 1), page, a.page_shift, blk, off);                     \
                KS_[i] = *(const uint4*)(kp + ((size_t)ATP_PAGE_OF(blk) * kv_stride + kvh_off + off * AT_HD + kpc[i])); \
            }                                                                                              \
        }                                                                                                  \
        _Pragma("unroll") for (int i = 0; i < ATP_VPT; ++i) {                                              \
            const int key4 = kb_ + vq[i];                                                                  \
            VS_[i] = make_uint2(0, 0);                                                                     \
            if (tid + 256 * i < ATP_VPIECES && key4 < key_hi) {                                            \
                int blk, off;                                                                              \
                split_key(key4, page, a.page_shift, blk, off);                                             \
                VS_[i] = keep_written(*(const uint2*)(vp + ((size_t)ATP_PAGE_OF(blk) * kv_stride + kvh_off + vd[i] * page + off)), key4, key_hi); \
            }                                                                                              \
        }                                                                                                  \
    }
#define ATP_PARK(KS_, VS_, buf)                                                                            \
    {                                                                                                      \
        _Pragma("unroll") for (int i = 0; i < ATP_KPT; ++i) {                                              \
            const int idx = tid + 256 * i;                                                                 \
            if (idx < ATP_KPIECES) *(uint4*)(&ks[buf][(idx / (AT_HD / 8)) * ATP_KROW + (idx % (AT_HD / 8)) * 8]) = KS_[i]; \
        }                                                                                                  \
        _Pragma("unroll") for (int i = 0; i < ATP_VPT; ++i) {                                              \
            const int idx = tid + 256 * i;                                                                 \
            if (idx < ATP_VPIECES) *(uint2*)(&vs[buf][(idx / 8) * ATP_VROW + (idx % 8) * 4]) = VS_[i];     \
        }                                                                                                  \
    }

    float m = -INFINITY, l = 0.f;
    f32x4_t acc[ATM_DT];
#pragma unroll
    for (int t = 0; t < ATM_DT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Pipeline: while chunk c is multiplied out of shared memory, chunk c+1 sits in registers
    // (fetched one iteration ago, parked at the end of this one) and chunk c+2 is being fetched:
    // a fetch has two iterations to arrive.
    if (ch_begin < ch_end) {
        ATP_FETCH(kst, vst, ch_begin)
        ATP_PARK(kst, vst, 0)
    }
    if (ch_begin + 1 < ch_end) ATP_FETCH(kst, vst, ch_begin + 1)
    __syncthreads();
    for (int ch = ch_begin; ch < ch_end; ++ch) {
        const int cur = (ch - ch_begin) & 1;
        const int kbase = ch * 32;
        if (ch + 2 < ch_end) ATP_FETCH(kst2, vst2, ch + 2)
        if (wave_has_rows && kbase <= w_pos_max && kbase + 31 >= w_lo_min) {
            f32x4_t sc[2];
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                f32x4_t sacc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int c = 0; c < ATM_DC; ++c) {
                    const int d = 32 * c + 8 * g;
                    FragK kf;
                    kf.u = (d + 8 <= AT_HD) ? *(const uint4*)(&ks[cur][(16 * hf + li) * ATP_KROW + d]) : make_uint4(0, 0, 0, 0);
                    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[c].v, sacc, 0, 0, 0);
                }
                sc[hf] = sacc;
            }
            float s[8];
            float mloc = -INFINITY;
            if (kbase + 31 <= w_pos_min && kbase >= w_lo_max) {
#pragma unroll
                for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float x = sc[hf][v] * scale2;
                        s[4 * hf + v] = x;
                        mloc = fmaxf(mloc, x);
                    }
            } else {
#pragma unroll
                for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int key = kbase + 16 * hf + 4 * g + v;
                        const bool seen = row_ok && key <= r_pos && key >= r_lo;
                        const float x = seen ? sc[hf][v] * scale2 : -INFINITY;
                        s[4 * hf + v] = x;
                        mloc = fmaxf(mloc, x);
                    }
            }
            mloc = max_across_halves(max_across_rows(mloc));
            const float m_new = fmaxf(m, mloc);
            const float alpha = (m == -INFINITY) ? 0.f : fast_exp2(m - m_new);
            FragK pf;
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float p = (s[i] == -INFINITY) ? 0.f : fast_exp2(s[i] - m_new);
                psum += p;
                pf.v[i] = (__bf16)p;
            }
            l = l * alpha + psum;
            const bool moved = __any(m_new != m);
            m = m_new;
#pragma unroll
            for (int t = 0; t < ATM_DT; ++t) {
                FragK vf;
                vf.h[0] = *(const uint2*)(&vs[cur][(16 * t + li) * ATP_VROW + 4 * g]);
                vf.h[1] = *(const uint2*)(&vs[cur][(16 * t + li) * ATP_VROW + 16 + 4 * g]);
                if (moved) acc[t] *= alpha;
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, acc[t], 0, 0, 0);
            }
        }
        if (ch + 1 < ch_end) ATP_PARK(kst, vst, cur ^ 1)
#pragma unroll
        for (int i = 0; i < ATP_KPT; ++i) kst[i] = kst2[i];
#pragma unroll
        for (int i = 0; i < ATP_VPT; ++i) vst[i] = vst2[i];
        // A barrier that waits for this wave's shared-memory traffic only: __syncthreads() would
        // also wait for the fetch of chunk c+2, which is meant to stay in flight across it.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
#undef ATP_FETCH
#undef ATP_PARK
#undef ATP_PAGE_OF
    l += __shfl_xor(l, 16, TL_WAVE);
    l += __shfl_xor(l, 32, TL_WAVE);
    if (!row_ok) return;
    bf16_t* o = (bf16_t*)a.out + (size_t)r_token * a.heads * AT_HD + (size_t)r_head * AT_HD;
    const float inv = 1.f / l;
#pragma unroll
    for (int t = 0; t < ATM_DT; ++t) {
        union { uint2 u; uint16_t e[4]; } pk;
#pragma unroll
        for (int v = 0; v < 4; ++v) pk.e[v] = from_float<bf16_t>(acc[t][v] * inv).bits;
        *(uint2*)(o + 16 * t + 4 * g) = pk.u;
    }
}
#endif

// out[row] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s over the parts of a row.
// A thread owns four neighbouring elements of a row, a work-group of 256 threads as many rows as
// fit; the parts are read eight at a time with all loads issued before the first use.
// Rows are (token, head) pairs: all of them, or those of the tokens listed in `tokens`.
#define ATG_TPR (AT_HD / 4)            // threads per row
#define ATG_RPW (256 / ATG_TPR)        // rows per work-group
template <typename T>
__global__ __launch_bounds__(256) void attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                              T* __restrict__ out, int splits, const int* __restrict__ tokens,
                                                              int heads, int rows, int hd) {
    const int local = threadIdx.x / ATG_TPR;
    const long listed = (long)blockIdx.x * ATG_RPW + local;
    if (local >= ATG_RPW || listed >= rows) return;
    const size_t r = tokens ? (size_t)tokens[listed / heads] * heads + listed % heads : (size_t)listed;
    const float2* ml = (const float2*)(part_ml + r * splits * 2);
    const float* po = part_o + r * splits * AT_HD;
    const int d = 4 * (threadIdx.x % ATG_TPR);
    float mx = -INFINITY, denom = 0.f;
    float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < splits; s0 += 8) {
        float2 w[8];
        float4 o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int sp = min(s0 + i, splits - 1);
            w[i] = ml[sp];
            o[i] = *(const float4*)(po + (size_t)sp * AT_HD + d);
        }
        float m8 = mx;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < splits) m8 = fmaxf(m8, w[i].x);
        const float rescale = (mx == -INFINITY) ? 0.f : expf(mx - m8);
        denom *= rescale;
        num.x *= rescale; num.y *= rescale; num.z *= rescale; num.w *= rescale;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < splits && w[i].x != -INFINITY) {
                const float e = expf(w[i].x - m8);
                denom += e * w[i].y;
                num.x += e * o[i].x; num.y += e * o[i].y; num.z += e * o[i].z; num.w += e * o[i].w;
            }
        mx = m8;
    }
    T* dst = out + r * hd + d;             // the parts are HD wide, a row of out holds the true head size
    if (d + 3 < hd) {
        dst[0] = from_float<T>(num.x / denom);
        dst[1] = from_float<T>(num.y / denom);
        dst[2] = from_float<T>(num.z / denom);
        dst[3] = from_float<T>(num.w / denom);
    } else if (d + 1 < hd) {               // head sizes are even
        dst[0] = from_float<T>(num.x / denom);
        dst[1] = from_float<T>(num.y / denom);
    }
}

static void launch_merge(const void* part_o, const void* part_ml, void* out, int splits, const void* tokens, int heads,
                         long rows, bool f32, hipStream_t stream, int hd = AT_HD) {
    dim3 grid((unsigned)((rows + ATG_RPW - 1) / ATG_RPW)), block(256);
    if (f32) attention_merge_kernel<float><<<grid, block, 0, stream>>>((const float*)part_o, (const float*)part_ml, (float*)out, splits, (const int*)tokens, heads, (int)rows, hd);
    else attention_merge_kernel<bf16_t><<<grid, block, 0, stream>>>((const float*)part_o, (const float*)part_ml, (bf16_t*)out, splits, (const int*)tokens, heads, (int)rows, hd);
}

// =====================================================================================
// Prompt portions, 128 rows per work-group (bfloat16, head size 64 or 128, pages of 8, 16, 32, ...
// tokens, sequences of up to ATM_BT_MAX pages).
//
// Four waves of 32 rows share steps of 64 keys.  Keys and transposed values of a step go from
// the pages straight into shared memory (global_load_lds_dwordx4, two buffers: the next step is
// on its way while this one is multiplied, and two work-groups share a compute unit), in 16-byte
// pieces whose slot within a row is exclusive-ored with the row number, so that the operand reads
// of sixteen neighbouring rows fall on all banks.  A tile's time is its number of steps times what
// a step takes from barrier to barrier, so steps of 64 keys beat steps of 32 with more of them in
// flight (28 heads in 4 groups, one MI355X: a prompt of 2048 tokens 86 -> 66 us, of 8192 tokens
// 648 -> 580 us = 0.83 PFLOP/s; steps of 64 keys with three or four buffers leave room for one
// work-group per compute unit only: 66 us at 2048 tokens but 779 us at 8192).
// Both products run transposed on v_mfma_f32_32x32x16_bf16:
//   S^T[key, row] = K[key, :] . Q[row, :]      A = 32 keys x 16 d from shared memory, B = Q (registers)
//   O^T[d, row]  += V^T[d, key] . P^T[key, row] A = 32 d x 16 keys from shared memory, B = P (registers)
// so a lane owns ONE query row (its column, lane % 32): maximum, sum and the rescaling of the
// accumulator are lane-local but for one exchange with lane ^ 32.  Which key an A row of the
// first product carries is free; row 8 q + 4 h + v carries key 16 (q / 2) + 8 h + 4 (q % 2) + v of
// its block of 32, which makes the eight probabilities a lane holds for a 16-key chunk exactly
// the B operand of the second product, with no exchange between lanes.
#if AT_HD == 64 || AT_HD == 128
#define ATQ_ROWS 128
#ifndef ATQ_KEYS
#define ATQ_KEYS 64                 // keys per step: 32 or 64
#endif
#ifndef ATQ_STAGES
#define ATQ_STAGES 2               // steps in shared memory: this one and those on their way
#endif
#define ATQ_KB (ATQ_KEYS / 32)      // blocks of 32 keys per step
#define ATQ_VROW (ATQ_KEYS * 2)     // bytes of a transposed value row (one d, the step's keys)
#define ATQ_VPP (ATQ_KEYS / 8)      // 16-byte pieces in it
#define ATQ_KBYTES (ATQ_KEYS * AT_HD * 2)
#define ATQ_STAGE (2 * ATQ_KBYTES)                 // keys, then values
#define ATQ_SMEM (ATQ_STAGES * ATQ_STAGE + ATM_BT_MAX * 4)
#define ATQ_SLACK 8.f               // powers of two a row's scores may rise above its reference before it is moved
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// 16 bytes per lane from memory straight into shared memory at lds_addr + 16 * lane.  Issued as
// assembly: the compiler would make every later shared-memory read wait for a direct load it
// knows of; the kernel waits itself (vmcnt) before the barrier that publishes a step.
__device__ __forceinline__ void attn_load_to_lds(const void* gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(gptr), "s"(lds_addr) : "memory", "m0");
}

// The same from a base that the wave shares plus 32 bits of each lane's own.
__device__ __forceinline__ void attn_load_to_lds_at(const void* base, unsigned offset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(offset), "s"(base), "s"(lds_addr) : "memory", "m0");
}

__device__ __forceinline__ int atq_key_slot(int piece, int key) {        // slot of a 16-byte piece in its key row
    return AT_HD == 128 ? (piece ^ (key & 15)) : (piece ^ ((key >> 1) & 7));
}
__device__ __forceinline__ int atq_value_slot(int piece, int d) {        // ... in its transposed value row
    return ATQ_KEYS == 64 ? (piece ^ ((d >> 1) & 7)) : (piece ^ ((d >> 2) & 3));
}

// LONG: pages of more than ATQ_KEYS keys, where a step begins inside a page (an addition per address that the usual
// short pages are spared).
template <bool LONG>
__global__ __launch_bounds__(256, 2) void paged_attention_prompt_kernel(AttnArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char atq_smem[];
    int* bt_s = (int*)(atq_smem + ATQ_STAGES * ATQ_STAGE);
    const unsigned lds_base = (unsigned)(uintptr_t)((void __attribute__((address_space(3)))*)atq_smem);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lr = lane & 31, h = lane >> 5;

    // Late tiles see the most keys: they start first, each with all its key/value heads, so that the
    // work-groups still running at the end are the light ones (launch order runs along x first; taking
    // the tile from x alone started the heavy tiles of the last head after the light ones of the first:
    // a 2048-token prompt 83 -> 75 us, 4096 tokens 231 -> 180 us, 2048 tokens with 40 heads in 8 groups
    // 102 -> 81 us).
    const int per_tile = gridDim.y;
    // With more work-groups than compute units, but no more than fit at once (two a unit), nothing is handed out
    // later to even things out: unit u runs the u-th work-group and the (units + u)-th, so the second batch
    // runs from light to heavy and every unit gets a heavy tile and a light one (2048 tokens, 28 heads in 4
    // groups, 256 units: 456 work-groups, 51 -> 49 us).
    int rank = blockIdx.y * gridDim.x + blockIdx.x;
    {
        const int n = gridDim.x * gridDim.y;
        if (gridDim.z == 1 && n <= 2 * a.units && rank >= a.units) rank = n - 1 - (rank - a.units);
    }
    const int tile = gridDim.x - 1 - rank / per_tile;
    const int by = rank % per_tile;
    const int group = a.heads / a.kv_heads;
    const int chunks_h = (group + a.gcap - 1) / a.gcap;
    const int kvh = by / chunks_h;
    const int g0 = (by % chunks_h) * a.gcap;
    const int gcount = min(a.gcap, group - g0);

    const int req = a.tile_req[tile];
    const int tok0 = a.tile_tok0[tile];
    const int first = a.req_indptr[req];
    const int n_new = a.req_indptr[req + 1] - first;
    const int ctx = a.ctx_lens[req];
    const int ntok = min(a.tq, n_new - tok0);

    const int row = wave * 32 + lr;
    const int r_tok = row / a.gcap, r_g = row % a.gcap;
    const bool row_ok = r_tok < ntok && r_g < gcount;
    const int r_pos = ctx + tok0 + r_tok;
    const int r_lo = a.window > 0 ? r_pos - a.window + 1 : 0;
    const int r_head = kvh * group + g0 + r_g;
    const int r_token = first + tok0 + r_tok;

    // the wave's rows: smallest and largest position, largest window start (uniform)
    const int w_tok_lo = min((wave * 32) / a.gcap, ntok - 1), w_tok_hi = min((wave * 32 + 31) / a.gcap, ntok - 1);
    const bool wave_has_rows = (wave * 32) / a.gcap < ntok;
    const int w_pos_min = ctx + tok0 + w_tok_lo, w_pos_max = ctx + tok0 + w_tok_hi;
    const int w_lo_min = a.window > 0 ? max(0, w_pos_min - a.window + 1) : 0;
    const int w_lo_max = a.window > 0 ? max(0, w_pos_max - a.window + 1) : 0;

    const int key_hi = ctx + tok0 + ntok;
    const int key_lo = a.window > 0 ? max(0, ctx + tok0 - a.window + 1) : 0;
    // the tile's steps of ATQ_KEYS keys; with a.splits > 1 work-group blockIdx.z takes its share of them
    // and leaves unnormalised sums, maxima and denominators for attention_merge_kernel
    int st_first = key_lo / ATQ_KEYS, st_last = (key_hi + ATQ_KEYS - 1) / ATQ_KEYS;
    if (a.splits > 1) {
        const int per = (st_last - st_first + a.splits - 1) / a.splits;
        st_first = min(st_first + (int)blockIdx.z * per, st_last);
        st_last = min(st_first + per, st_last);
    }

    const bf16_t* kp = (const bf16_t*)a.k_plane;
    const bf16_t* vp = (const bf16_t*)a.v_plane;
    const int page = a.page;
    const size_t kv_stride = (size_t)a.kv_heads * page * AT_HD;
    const int kvh_off = kvh * page * AT_HD;
    // the request's block-table row goes to shared memory (the host checked that it fits); pages are a
    // power of two, so a key's block and place in it are a shift and a mask
    const int* bt_g = a.block_table + (size_t)req * a.bt_stride;
    const int shift = a.page_shift, pmask = page - 1;
    const int blk0 = (st_first * ATQ_KEYS) >> shift;
    const int blk_n = ((key_hi - 1) >> shift) - blk0 + 1;
    if (blk_n > ATM_BT_MAX) return;            // longer than the host promised: leave the rows unwritten rather than overrun
    // A tile begins with three trips to memory: the block table, which the first requests need, those requests, and
    // the query.  The table is asked for first and the query right after it, so that the query is on its way while
    // the table arrives and the first keys and values are requested.
    const int bt_first = (int)threadIdx.x < blk_n ? bt_g[blk0 + threadIdx.x] : 0;
    // my row's query, B operand of the first product: d = 16 c + 8 h .. + 8
    FragK qf[AT_HD / 16];
    {
        const bf16_t* q = (const bf16_t*)a.q + (size_t)r_token * a.q_stride + (size_t)r_head * AT_HD;
#pragma unroll
        for (int c = 0; c < AT_HD / 16; ++c) qf[c].u = row_ok ? *(const uint4*)(q + 16 * c + 8 * h) : make_uint4(0, 0, 0, 0);
    }
    if ((int)threadIdx.x < blk_n) bt_s[threadIdx.x] = bt_first;
    for (int i = threadIdx.x + 256; i < blk_n; i += 256) bt_s[i] = bt_g[blk0 + i];
    __syncthreads();
    const bool any_step = st_first < st_last;  // (a share of the steps can be empty)

    // requests of one step: K rows of AT_HD * 2 bytes, then V^T rows of ATQ_VROW bytes
    constexpr int KPI = 1024 / (AT_HD * 2);                 // keys per load instruction (4 or 8)
    constexpr int KPP = AT_HD / 8;                          // pieces per key row (16 or 8)
    constexpr int K_INSTR = ATQ_KBYTES / 1024 / 4;          // per wave
    constexpr int VDI = 1024 / ATQ_VROW;                    // value rows (d) per load instruction (8 or 16)
    static_assert(K_INSTR >= 1 && 2 * K_INSTR * (ATQ_STAGES - 2) < 64, "loads per wave and step");
    // What does not change from step to step is worked out here, per load instruction of this lane: a step's first key
    // is a multiple of ATQ_KEYS, and pages are powers of two, so key kbase + x (x < ATQ_KEYS) lies in block
    // (kbase >> shift) + (x >> shift) at place (kbase & pmask) + (x & pmask) of its page (of the two uniform parts the
    // second is zero for pages of up to ATQ_KEYS keys, of the two lane parts the first is zero for longer ones).  A
    // step then costs a lane one look-up of a page and one multiply-add per address.  (With all of it computed in the
    // step, the addresses were a quarter of the loop's vector instructions.)
    // A page's keys (values) of all heads are kv_stride elements; the host checked that twice that fits 32 bits, so an
    // address is ONE 64-bit multiply-add of page number and stride on what was worked out here.
    // The keys of one load instruction (1024 bytes: 4 or 8 rows) lie in one page, pages being of 8 keys or more: their
    // page's address is the wave's, worked out by the scalar unit, and a lane adds 32 bits that never change.
    unsigned k_off[K_INSTR];                   // K row of key x, this lane's piece: bytes from the start of its head's page
    unsigned long long v_src[K_INSTR];         // V^T row d, this lane's eight keys, in page 0
    int k_blk[K_INSTR];                        // x >> shift
    unsigned k_dst[K_INSTR];
    int v_blk;                                 // the same for every value load of a lane (its piece's slot depends on d / 2 mod 8 only)
#pragma unroll
    for (int j = 0; j < K_INSTR; ++j) {
        const int ii = wave + 4 * j;
        const int kx = KPI * ii + lane / KPP;
        k_blk[j] = kx >> shift;
        k_off[j] = (unsigned)((kx & pmask) * AT_HD + atq_key_slot(lane % KPP, kx) * 8) * 2u;       // exclusive-or is its own inverse
        const int d = VDI * ii + lane / ATQ_VPP;
        const int vx = 8 * atq_value_slot(lane % ATQ_VPP, d);           // first of the piece's eight keys
        if (j == 0) v_blk = vx >> shift;
        v_src[j] = (unsigned long long)(uintptr_t)(vp + kvh_off + d * page + (vx & pmask));
        k_dst[j] = __builtin_amdgcn_readfirstlane(ii * 1024);
    }
    const int blk_last = blk_n - 1;
    const unsigned page_bytes = (unsigned)kv_stride * 2u;
    // The pages of a step are looked up one request early and kept in registers: looked up where they are needed, each
    // of the five look-ups stood between a request and the one before it, with the trip to shared memory in full.
    // (a block beyond the sequence's last is read as the last: the step that holds the sequence's end may reach past
    // its last page; those keys' scores are masked and their values cleared below)
    // Look-ups and requests come one at a time (j: the step's K_INSTR key loads, then its value loads), for the loop
    // to place them between its products.
    int pg_k[K_INSTR], pg_v;
    auto look_up_one = [&](int st, int j) {
        const int ub = ((st * ATQ_KEYS) >> shift) - blk0;                // uniform: the step's first block in bt_s
        if (j < K_INSTR) pg_k[j] = bt_s[min(ub + k_blk[j], blk_last)];
        else pg_v = bt_s[min(ub + v_blk, blk_last)];
    };
    auto look_up = [&](int st) {
#pragma unroll
        for (int j = 0; j <= K_INSTR; ++j) look_up_one(st, j);
    };
    auto request_one = [&](int st, int buf, int j) {                    // (after look_up(st))
        const unsigned sb = lds_base + buf * ATQ_STAGE;
        const unsigned uin = LONG ? (st * ATQ_KEYS) & pmask : 0;         // uniform: the step's first key's place in its page
        if (j < K_INSTR) {
            const unsigned pg = __builtin_amdgcn_readfirstlane(pg_k[j]);
            const unsigned long long src = (unsigned long long)(uintptr_t)(kp + kvh_off) + (unsigned long long)pg * page_bytes + uin * (AT_HD * 2);
            attn_load_to_lds_at((const void*)(uintptr_t)src, k_off[j], sb + k_dst[j]);
        } else {
            const unsigned long long v_page = (unsigned long long)(unsigned)pg_v * page_bytes + uin * 2;
            attn_load_to_lds((const void*)(uintptr_t)(v_src[j - K_INSTR] + v_page), sb + ATQ_KBYTES + k_dst[j - K_INSTR]);
        }
    };
    auto request_step = [&](int st, int buf) {
#pragma unroll
        for (int j = 0; j < 2 * K_INSTR; ++j) request_one(st, buf, j);
    };

    const float scale2 = a.scale * 1.44269504088896341f;
    float m = -INFINITY, l = 0.f;
    f32x16_t acc[AT_HD / 32];
#pragma unroll
    for (int b = 0; b < AT_HD / 32; ++b)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[b][v] = 0.f;

    // key (within its block of 32) that A row lr of the first product carries
    const int krow = 16 * (lr >> 4) + 8 * ((lr >> 2) & 1) + 4 * ((lr >> 3) & 1) + (lr & 3);

    // Steps st .. st + ATQ_STAGES - 2 are requested ahead; past the end the last step is requested
    // again (nobody reads it), so that the number of requests in flight is the same at every wait.
    if (any_step) {
#pragma unroll
        for (int i = 0; i < ATQ_STAGES - 1; ++i) {
            look_up(min(st_first + i, st_last - 1));
            request_step(min(st_first + i, st_last - 1), i);
        }
        look_up(min(st_first + ATQ_STAGES - 1, st_last - 1));
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * K_INSTR * (ATQ_STAGES - 2)) : "memory");
        __syncthreads();
    }
    // The query is waited for here, once.  Left to the compiler, the wait would stand before the first product of
    // every step (at the loop's head it must assume the fetch of before the loop still under way), and as a wait for
    // all fetches it would also wait for the keys and values just requested for the next step: no step would
    // overlap with the fetch of the next.
#pragma unroll
    for (int c = 0; c < AT_HD / 16; ++c) asm volatile("" : "+v"(qf[c].v));
    for (int st = st_first; st < st_last; ++st) {
        const int buf = (st - st_first) % ATQ_STAGES;
        const int st_req = min(st + ATQ_STAGES - 1, st_last - 1), buf_req = (st - st_first + ATQ_STAGES - 1) % ATQ_STAGES;
        const int st_look = min(st + ATQ_STAGES, st_last - 1);
        const int kbase = st * ATQ_KEYS;
        unsigned char* kb_s = atq_smem + buf * ATQ_STAGE;
        unsigned char* vb_s = kb_s + ATQ_KBYTES;
        if (kbase + ATQ_KEYS > key_hi) {
            // the last step holds keys that are not written yet: whatever lies in their places in
            // the pages must not reach the second product (0 * Inf), so their values become zero
            for (int i = threadIdx.x; i < AT_HD * ATQ_VPP; i += 256) {
                const int d = i / ATQ_VPP, piece = i % ATQ_VPP;
                const int k0 = kbase + 8 * piece;
                if (k0 + 8 > key_hi) {
                    FragK f;
                    uint4* ptr = (uint4*)(vb_s + d * ATQ_VROW + atq_value_slot(piece, d) * 16);
                    f.u = *ptr;
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (k0 + e >= key_hi) f.v[e] = (__bf16)0.f;
                    *ptr = f.u;
                }
            }
            __syncthreads();
        }
        if (wave_has_rows && kbase <= w_pos_max && kbase + ATQ_KEYS > w_lo_min) {
            // ---- scores of two blocks of 32 keys
            // (the blocks take turns: a product that adds to the sums of the one before it waits for it to finish)
            f32x16_t sc[ATQ_KB];
#pragma unroll
            for (int kb = 0; kb < ATQ_KB; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) sc[kb][v] = 0.f;
            // and a block's keys are read two products of that block ahead
            constexpr int KAHEAD = 2;
            FragK kf[KAHEAD + 1][ATQ_KB];
            auto read_keys = [&](int c, int kb) {
                const int kl = 32 * kb + krow;
                kf[c % (KAHEAD + 1)][kb].u = *(const uint4*)(kb_s + kl * (AT_HD * 2) + atq_key_slot(2 * c + h, kl) * 16);
            };
#pragma unroll
            for (int c = 0; c < KAHEAD; ++c)
#pragma unroll
                for (int kb = 0; kb < ATQ_KB; ++kb) read_keys(c, kb);
            __builtin_amdgcn_sched_barrier(0);
            // (the requests of the step ahead go between the products, one beside every other product)
            static_assert(AT_HD / 16 * ATQ_KB >= 4 * K_INSTR, "a request beside every other product");
#pragma unroll
            for (int c = 0; c < AT_HD / 16; ++c)
#pragma unroll
                for (int kb = 0; kb < ATQ_KB; ++kb) {
                    sc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[c % (KAHEAD + 1)][kb].v, qf[c].v, sc[kb], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    if (c + KAHEAD < AT_HD / 16) read_keys(c + KAHEAD, kb);
                    const int slot = c * ATQ_KB + kb;
                    if (slot % 2 == 0 && slot / 2 < 2 * K_INSTR) request_one(st_req, buf_req, slot / 2);
                    __builtin_amdgcn_sched_barrier(0);
                }
            // ---- mask, maximum, probabilities.  Element (kb, 4 q + v) of this lane is key
            // kbase + 32 kb + 16 (q / 2) + 8 h + 4 (q % 2) + v of row lr.  The maximum is taken of the scores as
            // they come out of the product; the factor on them (positive: the host checks) goes into the
            // exponent's argument, one multiply-add per score.
            float mloc = -INFINITY;
            if (kbase + ATQ_KEYS - 1 <= w_pos_min && kbase >= w_lo_max) {
#pragma unroll
                for (int kb = 0; kb < ATQ_KB; ++kb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) mloc = fmaxf(mloc, sc[kb][v]);
            } else {
#pragma unroll
                for (int kb = 0; kb < ATQ_KB; ++kb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int q = e >> 2, v = e & 3;
                        const int key = kbase + 32 * kb + 16 * (q >> 1) + 8 * h + 4 * (q & 1) + v;
                        const bool seen = row_ok && key <= r_pos && key >= r_lo;
                        sc[kb][e] = seen ? sc[kb][e] : -INFINITY;
                        mloc = fmaxf(mloc, sc[kb][e]);
                    }
            }
            mloc = max_across_halves(mloc) * scale2;
            // m is the row's reference for the exponents, not its running maximum: it moves only when some row of
            // the wave has a score more than ATQ_SLACK (in powers of two) above its reference, so most steps rescale
            // nothing; until then probabilities are up to 2^ATQ_SLACK instead of up to 1, which 32-bit sums and the
            // bfloat16 operand of the second product hold as exactly as before, and the quotient at the end is the same.
            if (__any(mloc > m + ATQ_SLACK)) {
                const float m_new = fmaxf(m, mloc);
                const float alpha = (m == -INFINITY) ? 0.f : fast_exp2(m - m_new);      // 1 for a row that stays
                m = m_new;
                l *= alpha;
#pragma unroll
                for (int b = 0; b < AT_HD / 32; ++b) acc[b] *= alpha;
            }
            const float m_use = (m == -INFINITY) ? 0.f : -m;           // nothing seen yet: every score is -inf
            FragK pf[2 * ATQ_KB];
            float psum = 0.f;
            auto probabilities = [&](int kb, int e0, int n) {
#pragma unroll
                for (int e = e0; e < e0 + n; ++e) {
                    const float p = fast_exp2(__builtin_fmaf(sc[kb][e], scale2, m_use));
                    psum += p;
                    pf[2 * kb + (e >> 3)].v[e & 7] = (__bf16)p;
                }
            };
            // ---- values.  Product i takes the values of d = 32 (i % NB) .. + 32 for the 16 keys of chunk i / NB; the
            // values are read two products ahead.  Only the first block's probabilities are worked out before the
            // products begin: those of each later block go beside the products of the block before it, and the
            // look-ups of the pages that the next step requests beside the products of the last block, so that the
            // vector unit works while the matrix unit does.
            constexpr int NB = AT_HD / 32, NPV = 2 * ATQ_KB * NB, VAHEAD = 2;
            constexpr int PER = 16 / (2 * NB);                     // probabilities beside one product
            static_assert(2 * NB >= K_INSTR + 1, "a look-up beside each product of the last block");
            FragK vfb[VAHEAD + 1];
            auto read_values = [&](int i) {
                const int d = 32 * (i % NB) + lr;
                vfb[i % (VAHEAD + 1)].u = *(const uint4*)(vb_s + d * ATQ_VROW + atq_value_slot(2 * (i / NB) + h, d) * 16);
            };
#pragma unroll
            for (int i = 0; i < VAHEAD; ++i) read_values(i);
            probabilities(0, 0, 16);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < NPV; ++i) {
                acc[i % NB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfb[i % (VAHEAD + 1)].v, pf[i / NB].v, acc[i % NB], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (i + VAHEAD < NPV) read_values(i + VAHEAD);
                const int kb = i / (2 * NB), within = i % (2 * NB);
                if (kb + 1 < ATQ_KB) probabilities(kb + 1, within * PER, PER);
                else if (within <= K_INSTR) look_up_one(st_look, within);
                __builtin_amdgcn_sched_barrier(0);
            }
            l += psum;
        } else {
            request_step(st_req, buf_req);
            look_up(st_look);
        }
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * K_INSTR * (ATQ_STAGES - 2)) : "memory");
        __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    l += __shfl_xor(l, 32, TL_WAVE);
    if (!row_ok) return;
    // lane holds d = 32 b + 8 q + 4 h + v of its row
    if (a.splits > 1) {
        const size_t pr = ((size_t)r_token * a.heads + r_head) * a.splits + blockIdx.z;
        float* po = a.part_o + pr * AT_HD;
#pragma unroll
        for (int b = 0; b < AT_HD / 32; ++b)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                f32x4_t f;
#pragma unroll
                for (int v = 0; v < 4; ++v) f[v] = acc[b][4 * q + v];
                *(f32x4_t*)(po + 32 * b + 8 * q + 4 * h) = f;
            }
        if (h == 0) {
            a.part_ml[pr * 2] = m * 0.69314718055994531f;      // back to natural logarithms for the merge
            a.part_ml[pr * 2 + 1] = l;
        }
        return;
    }
    bf16_t* o = (bf16_t*)a.out + (size_t)r_token * a.heads * AT_HD + (size_t)r_head * AT_HD;
    const float inv = 1.f / l;
#pragma unroll
    for (int b = 0; b < AT_HD / 32; ++b)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            union { uint2 u; uint16_t e[4]; } pk;
#pragma unroll
            for (int v = 0; v < 4; ++v) pk.e[v] = from_float<bf16_t>(acc[b][4 * q + v] * inv).bits;
            *(uint2*)(o + 32 * b + 8 * q + 4 * h) = pk.u;
        }
}
#endif

// The 128-row prompt kernel: tiles of `tq` tokens with tq * min(group, 128) <= 128.  Returns an
// error where it is not built (head sizes other than 64 and 128, pages that are no power of two from 8 up,
// sequences longer than tl_paged_attention_prompt_blocks() pages).
extern "C" int tl_paged_attention_prompt_rows() {
#if AT_HD == 64 || AT_HD == 128
    return ATQ_ROWS;
#else
    return 0;
#endif
}

extern "C" int tl_paged_attention_prompt_blocks() { return ATM_BT_MAX; }

extern "C" int tl_paged_attention_prompt(const void* q, int q_stride, void* out, const void* k_plane, const void* v_plane,
                                         const void* block_table, int bt_stride, const void* req_indptr, const void* ctx_lens,
                                         const void* tile_req, const void* tile_tok0, int tiles, int tq,
                                         int heads, int kv_heads, int page, int window, float scale, int used_blocks,
                                         int splits, void* part_o, void* part_ml, const void* merge_tokens, int merge_count,
                                         hipStream_t stream) {
    // splits > 1: every tile's keys are dealt to that many work-groups, whose parts (scratch as for
    // tl_paged_attention) are merged for the `merge_count` tokens listed in `merge_tokens`: for prompt
    // portions whose tiles alone leave most compute units idle.
#if AT_HD == 64 || AT_HD == 128
    TL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "attention: heads %d not a multiple of kv heads %d", heads, kv_heads);
    TL_REQUIRE(page >= 8 && (page & (page - 1)) == 0 && tq > 0 && window >= 0, "attention_prompt: pages of 8, 16, 32, ... tokens, not %d", page);
    TL_REQUIRE(scale > 0.f, "attention_prompt: the factor on the scores must be positive (the maximum is taken before it is applied), not %g", (double)scale);
    // used_blocks: the most block-table entries any request of the step uses (its length in pages)
    TL_REQUIRE(bt_stride > 0 && used_blocks > 0 && used_blocks <= ATM_BT_MAX,
               "attention_prompt: sequences of up to %d pages, not %d", ATM_BT_MAX, used_blocks);
    TL_REQUIRE((long)kv_heads * page * AT_HD * 2 < (1L << 32), "attention_prompt: a page of %d heads x %d tokens is too large", kv_heads, page);
    const int group = heads / kv_heads;
    const int gcap = group < ATQ_ROWS ? group : ATQ_ROWS;
    TL_REQUIRE(tq * gcap <= ATQ_ROWS, "attention_prompt: tile of %d tokens x %d heads exceeds %d rows", tq, gcap, ATQ_ROWS);
    TL_REQUIRE(q_stride >= heads * AT_HD && q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 &&
               ((uintptr_t)k_plane % 16) == 0 && ((uintptr_t)v_plane % 16) == 0, "attention_prompt: operands not aligned");
    if (tiles == 0) return TL_OK;
    AttnArgs a;
    a.q = q; a.out = out; a.k_plane = k_plane; a.v_plane = v_plane;
    a.block_table = (const int*)block_table; a.req_indptr = (const int*)req_indptr; a.ctx_lens = (const int*)ctx_lens;
    a.tile_req = (const int*)tile_req; a.tile_tok0 = (const int*)tile_tok0;
    TL_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || (part_o && part_ml && merge_tokens && merge_count > 0)),
               "attention_prompt: splits > 1 need scratch and the tokens to merge");
    a.part_o = (float*)part_o; a.part_ml = (float*)part_ml;
    a.q_stride = q_stride; a.bt_stride = bt_stride; a.heads = heads; a.kv_heads = kv_heads; a.page = page;
    a.window = window; a.tq = tq; a.gcap = gcap; a.splits = splits; a.scale = scale; a.hd = AT_HD;
    a.page_shift = (page & (page - 1)) == 0 ? __builtin_ctz(page) : -1;
    static int units = 0;                        // (of the device of the first call: one kind of GPU in a process)
    if (units == 0) {
        int dev = 0, n = 0;
        TL_REQUIRE(hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0,
                   "attention_prompt: cannot ask the device for its compute units");
        units = n;
    }
    a.units = units;
    const int chunks = (group + gcap - 1) / gcap;
    static hipError_t allowed = hipFuncSetAttribute((const void*)paged_attention_prompt_kernel<false>,
                                                    hipFuncAttributeMaxDynamicSharedMemorySize, ATQ_SMEM);
    static hipError_t allowed_long = hipFuncSetAttribute((const void*)paged_attention_prompt_kernel<true>,
                                                         hipFuncAttributeMaxDynamicSharedMemorySize, ATQ_SMEM);
    TL_REQUIRE(allowed == hipSuccess && allowed_long == hipSuccess, "attention_prompt: cannot get %d bytes of shared memory", ATQ_SMEM);
    if (page > ATQ_KEYS) paged_attention_prompt_kernel<true><<<dim3(tiles, kv_heads * chunks, splits), dim3(256), ATQ_SMEM, stream>>>(a);
    else paged_attention_prompt_kernel<false><<<dim3(tiles, kv_heads * chunks, splits), dim3(256), ATQ_SMEM, stream>>>(a);
    TL_CHECK_LAUNCH("paged_attention_prompt");
    if (splits > 1) {
        launch_merge(part_o, part_ml, out, splits, merge_tokens, heads, (long)merge_count * heads, false, stream);
        TL_CHECK_LAUNCH("attention_merge");
    }
    return TL_OK;
#else
    TL_REQUIRE(false, "attention_prompt: built for head sizes 64 and 128, this library is for %d", AT_HD);
#endif
}

extern "C" int tl_attention_head_dim() { return AT_HD; }

// Scratch the caller must provide when splits > 1:
//   part_o  float[tokens * heads * splits * HD], part_ml float[tokens * heads * splits * 2].
extern "C" int tl_paged_attention(const void* q, int q_stride, void* out, const void* k_plane, const void* v_plane,
                                  const void* block_table, int bt_stride, const void* req_indptr, const void* ctx_lens,
                                  const void* tile_req, const void* tile_tok0, int tiles, int tokens, int tq,
                                  int heads, int kv_heads, int head_dim, int page, int window, float scale, int splits,
                                  void* part_o, void* part_ml, const void* merge_tokens, int merge_count, int dtype, int general,
                                  int waves, hipStream_t stream) {
    TL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "attention: heads %d not a multiple of kv heads %d", heads, kv_heads);
    TL_REQUIRE(waves == 4 || waves == 8, "attention: work-groups of 4 or 8 waves, not %d", waves);
    TL_REQUIRE(head_dim > AT_HD - 16 && head_dim <= AT_HD && head_dim % 2 == 0,
               "attention: this library serves the even head sizes %d to %d, not %d", AT_HD - 14, AT_HD, head_dim);
    TL_REQUIRE(page > 0 && bt_stride > 0 && tq > 0 && splits > 0 && window >= 0, "attention: bad page/table/tile sizes");
    TL_REQUIRE(splits == 1 || (part_o && part_ml), "attention: splits > 1 needs scratch");
    TL_REQUIRE((tile_req && tile_tok0 && req_indptr) || (!tile_req && !tile_tok0 && tiles == tokens),
               "attention: without a tile list every request brings one token (tiles %d, tokens %d)", tiles, tokens);
    const int group = heads / kv_heads;
    const int gcap = group < AT_ROWS ? group : AT_ROWS;
    TL_REQUIRE(tq * gcap <= AT_ROWS, "attention: tile of %d tokens x %d heads exceeds %d rows", tq, gcap, AT_ROWS);
    TL_REQUIRE(q_stride >= heads * head_dim, "attention: q stride %d too small", q_stride);
    if (tiles == 0 || tokens == 0) return TL_OK;
    AttnArgs a;
    a.q = q; a.out = out; a.k_plane = k_plane; a.v_plane = v_plane;
    a.block_table = (const int*)block_table; a.req_indptr = (const int*)req_indptr; a.ctx_lens = (const int*)ctx_lens;
    a.tile_req = (const int*)tile_req; a.tile_tok0 = (const int*)tile_tok0;
    a.part_o = (float*)part_o; a.part_ml = (float*)part_ml;
    a.q_stride = q_stride; a.bt_stride = bt_stride; a.heads = heads; a.kv_heads = kv_heads; a.page = page;
    a.window = window; a.tq = tq; a.gcap = gcap; a.splits = splits; a.scale = scale; a.hd = head_dim;
    a.page_shift = (page & (page - 1)) == 0 ? __builtin_ctz(page) : -1;
    const int chunks = (group + gcap - 1) / gcap;
    dim3 grid(tiles, kv_heads * chunks, splits), block(256);
    const bool aligned = ((uintptr_t)q % 16) == 0 && q_stride % 8 == 0 && ((uintptr_t)out % 8) == 0 &&
                         ((uintptr_t)k_plane % 16) == 0 && ((uintptr_t)v_plane % 8) == 0;
    if (dtype == TL_DT_F32) paged_attention_kernel<float><<<grid, block, 0, stream>>>(a);
    else if (dtype == TL_DT_BF16 && page % 4 == 0 && aligned && !general && head_dim == AT_HD) {
        if (waves == 8) paged_attention_mfma_kernel<8><<<grid, dim3(512), 0, stream>>>(a);
        else paged_attention_mfma_kernel<4><<<grid, block, 0, stream>>>(a);
    }
    else if (dtype == TL_DT_BF16) paged_attention_kernel<bf16_t><<<grid, block, 0, stream>>>(a);
    else TL_REQUIRE(false, "attention: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("paged_attention");
    if (splits > 1) {
        // merge_tokens: the tokens whose rows the tiles cover, when these are not all tokens of the step
        const size_t rows = (size_t)(merge_tokens ? merge_count : tokens) * heads;
        if (rows == 0) return TL_OK;
        launch_merge(part_o, part_ml, out, splits, merge_tokens, heads, (long)rows, dtype == TL_DT_F32, stream, head_dim);
        TL_CHECK_LAUNCH("attention_merge");
    }
    return TL_OK;
}

// Rows of a prompt-portion tile: a.tq tokens x gcap heads must fit 64.
#define ATP_ROWS 64

// The prompt-portion kernel (bfloat16, head sizes up to 128, pages of a multiple of 4 tokens):
// tiles of `tq` tokens with tq * min(group, 16) <= 64.  Returns an error where it is not built;
// callers fall back to tl_paged_attention, which takes every case.
extern "C" int tl_paged_attention_prefill(const void* q, int q_stride, void* out, const void* k_plane, const void* v_plane,
                                          const void* block_table, int bt_stride, const void* req_indptr, const void* ctx_lens,
                                          const void* tile_req, const void* tile_tok0, int tiles, int tq,
                                          int heads, int kv_heads, int page, int window, float scale, hipStream_t stream) {
#if AT_HD <= 128
    TL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "attention: heads %d not a multiple of kv heads %d", heads, kv_heads);
    TL_REQUIRE(page > 0 && page % 4 == 0 && bt_stride > 0 && tq > 0 && window >= 0, "attention_prefill: bad page/table/tile sizes");
    const int group = heads / kv_heads;
    const int gcap = group < AT_ROWS ? group : AT_ROWS;
    TL_REQUIRE(tq * gcap <= ATP_ROWS, "attention_prefill: tile of %d tokens x %d heads exceeds %d rows", tq, gcap, ATP_ROWS);
    TL_REQUIRE(q_stride >= heads * AT_HD && q_stride % 8 == 0 && ((uintptr_t)q % 16) == 0 && ((uintptr_t)out % 8) == 0 &&
               ((uintptr_t)k_plane % 16) == 0 && ((uintptr_t)v_plane % 8) == 0, "attention_prefill: operands not aligned");
    if (tiles == 0) return TL_OK;
    AttnArgs a;
    a.q = q; a.out = out; a.k_plane = k_plane; a.v_plane = v_plane;
    a.block_table = (const int*)block_table; a.req_indptr = (const int*)req_indptr; a.ctx_lens = (const int*)ctx_lens;
    a.tile_req = (const int*)tile_req; a.tile_tok0 = (const int*)tile_tok0;
    a.part_o = nullptr; a.part_ml = nullptr;
    a.q_stride = q_stride; a.bt_stride = bt_stride; a.heads = heads; a.kv_heads = kv_heads; a.page = page;
    a.window = window; a.tq = tq; a.gcap = gcap; a.splits = 1; a.scale = scale; a.hd = AT_HD;
    a.page_shift = (page & (page - 1)) == 0 ? __builtin_ctz(page) : -1;
    const int chunks = (group + gcap - 1) / gcap;
    paged_attention_prefill_kernel<<<dim3(tiles, kv_heads * chunks), dim3(256), 0, stream>>>(a);
    TL_CHECK_LAUNCH("paged_attention_prefill");
    return TL_OK;
#else
    TL_REQUIRE(false, "attention_prefill: built for head sizes up to 128, this library is for %d", AT_HD);
#endif
}
