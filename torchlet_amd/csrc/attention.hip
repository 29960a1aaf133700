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
// Compiled per head size: -DTL_HEAD_DIM=<multiple of 16>.
#include "common.h"

#ifndef TL_HEAD_DIM
#error "compile with -DTL_HEAD_DIM=<head size>"
#endif
static_assert(TL_HEAD_DIM % 16 == 0 && TL_HEAD_DIM >= 16 && TL_HEAD_DIM <= 512, "head size: multiple of 16 up to 512");

#define AT_ROWS 16
#define AT_HD TL_HEAD_DIM
#define AT_KT (AT_HD <= 128 ? 32 : (AT_HD <= 256 ? 16 : 8))   // keys per tile
#define AT_DPT (AT_HD / 16)                                   // output dims per thread

struct AttnArgs {
    const void* q;            // [tokens, q_stride], head h at column h * HD
    void* out;                // [tokens, heads * HD]
    const void* k_plane;      // [pages, kv_heads, page, HD]
    const void* v_plane;
    const int* block_table;   // [requests, bt_stride]
    const int* req_indptr;    // [requests + 1] first new token of each request
    const int* ctx_lens;      // [requests] tokens cached before this step
    const int* tile_req;      // [tiles]
    const int* tile_tok0;     // [tiles] first new token of the tile, relative to its request
    float* part_o;            // [tokens * heads, splits, HD] (splits > 1)
    float* part_ml;           // [tokens * heads, splits, 2]
    int q_stride, bt_stride, heads, kv_heads, page, window, tq, gcap, splits;
    float scale;
};

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

    const int req = a.tile_req[tile];
    const int tok0 = a.tile_tok0[tile];
    const int first = a.req_indptr[req];
    const int n_new = a.req_indptr[req + 1] - first;
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
        if (tt < ntok && gg < gcount)
            v = to_float(q[(size_t)(first + tok0 + tt) * a.q_stride + (size_t)(kvh * group + g0 + gg) * AT_HD + d]);
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
            if (pos < key_hi) {
                const int pg = bt[pos / a.page];
                const size_t off = (((size_t)pg * a.kv_heads + kvh) * a.page + (pos % a.page)) * AT_HD + d;
                kv = to_float(kp[off]);
                vv = to_float(vp[off]);
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
        T* o = (T*)a.out + (size_t)r_token * a.heads * AT_HD + (size_t)r_head * AT_HD;
        const float inv = 1.f / l;
#pragma unroll
        for (int i = 0; i < AT_DPT; ++i) o[sub + 16 * i] = from_float<T>(acc[i] * inv);
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

// out[row] = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s over the parts of a row.
template <typename T>
__global__ void attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                       T* __restrict__ out, int splits) {
    const size_t r = blockIdx.x;
    const float* ml = part_ml + r * splits * 2;
    float mx = -INFINITY;
    for (int s = 0; s < splits; ++s) mx = fmaxf(mx, ml[2 * s]);
    float denom = 0.f;
    for (int s = 0; s < splits; ++s)
        if (ml[2 * s] != -INFINITY) denom += expf(ml[2 * s] - mx) * ml[2 * s + 1];
    for (int d = threadIdx.x; d < AT_HD; d += blockDim.x) {
        float num = 0.f;
        for (int s = 0; s < splits; ++s)
            if (ml[2 * s] != -INFINITY) num += expf(ml[2 * s] - mx) * part_o[(r * splits + s) * AT_HD + d];
        out[r * AT_HD + d] = from_float<T>(num / denom);
    }
}

extern "C" int tl_attention_head_dim() { return AT_HD; }

// Scratch the caller must provide when splits > 1:
//   part_o  float[tokens * heads * splits * HD], part_ml float[tokens * heads * splits * 2].
extern "C" int tl_paged_attention(const void* q, int q_stride, void* out, const void* k_plane, const void* v_plane,
                                  const void* block_table, int bt_stride, const void* req_indptr, const void* ctx_lens,
                                  const void* tile_req, const void* tile_tok0, int tiles, int tokens, int tq,
                                  int heads, int kv_heads, int page, int window, float scale, int splits,
                                  void* part_o, void* part_ml, int dtype, hipStream_t stream) {
    TL_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "attention: heads %d not a multiple of kv heads %d", heads, kv_heads);
    TL_REQUIRE(page > 0 && bt_stride > 0 && tq > 0 && splits > 0 && window >= 0, "attention: bad page/table/tile sizes");
    TL_REQUIRE(splits == 1 || (part_o && part_ml), "attention: splits > 1 needs scratch");
    const int group = heads / kv_heads;
    const int gcap = group < AT_ROWS ? group : AT_ROWS;
    TL_REQUIRE(tq * gcap <= AT_ROWS, "attention: tile of %d tokens x %d heads exceeds %d rows", tq, gcap, AT_ROWS);
    TL_REQUIRE(q_stride >= heads * AT_HD, "attention: q stride %d too small", q_stride);
    if (tiles == 0 || tokens == 0) return TL_OK;
    AttnArgs a;
    a.q = q; a.out = out; a.k_plane = k_plane; a.v_plane = v_plane;
    a.block_table = (const int*)block_table; a.req_indptr = (const int*)req_indptr; a.ctx_lens = (const int*)ctx_lens;
    a.tile_req = (const int*)tile_req; a.tile_tok0 = (const int*)tile_tok0;
    a.part_o = (float*)part_o; a.part_ml = (float*)part_ml;
    a.q_stride = q_stride; a.bt_stride = bt_stride; a.heads = heads; a.kv_heads = kv_heads; a.page = page;
    a.window = window; a.tq = tq; a.gcap = gcap; a.splits = splits; a.scale = scale;
    const int chunks = (group + gcap - 1) / gcap;
    dim3 grid(tiles, kv_heads * chunks, splits), block(256);
    if (dtype == TL_DT_F32) paged_attention_kernel<float><<<grid, block, 0, stream>>>(a);
    else if (dtype == TL_DT_BF16) paged_attention_kernel<bf16_t><<<grid, block, 0, stream>>>(a);
    else TL_REQUIRE(false, "attention: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("paged_attention");
    if (splits > 1) {
        dim3 mgrid((unsigned)((size_t)tokens * heads)), mblock(AT_HD < 64 ? 64 : (AT_HD > 256 ? 256 : AT_HD));
        if (dtype == TL_DT_F32) attention_merge_kernel<float><<<mgrid, mblock, 0, stream>>>((const float*)part_o, (const float*)part_ml, (float*)out, splits);
        else attention_merge_kernel<bf16_t><<<mgrid, mblock, 0, stream>>>((const float*)part_o, (const float*)part_ml, (bf16_t*)out, splits);
        TL_CHECK_LAUNCH("attention_merge");
    }
    return TL_OK;
}
