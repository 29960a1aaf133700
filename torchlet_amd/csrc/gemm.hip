// Matrix products out[M, N] = x[M, K] * w[N, K]^T (+ bias[N]).
//
// Both operands are row-major with K contiguous, which is how activations and
// nn.Linear-layout weights are stored.  This file holds the general kernel: a 64x64 or 128x128
// tile, 256 threads with a 4x4 or 8x8 micro-tile each, products and sums in true 32-bit
// (v_fma_f32; no matrix-core instruction of reduced precision).  It is the matrix
// product of the 32-bit path and the fallback of the bfloat16 path for shapes that
// the matrix-core kernels refuse.  The sum over K runs in one fixed order for every
// output element, whatever M is, so a row's result does not depend on the batch.
#include "common.h"

// The compute units of the GPU the library runs on: the caller tells it once (tl_gemm_set_compute_units, from
// the device's properties); 256, the MI355X on which every plan below was measured, until it does.
static int g_compute_units = 256;
extern "C" void tl_gemm_set_compute_units(int n) { if (n > 0) g_compute_units = n; }
extern "C" int tl_gemm_compute_units() { return g_compute_units; }
#define TL_COMPUTE_UNITS g_compute_units


#define GT_K 16

// BT x BT tile, 256 threads with a (BT / 16) x (BT / 16) micro-tile each: 64 x 64 for small products,
// 128 x 128 (64 products per thread and K step against four 16-byte reads of shared memory) for
// large ones.  Both add the products of an output element in the same order, k = 0, 1, 2, ...
template <typename TIn, typename TOut, int BT>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const TIn* __restrict__ x, const TIn* __restrict__ w,
                                                        const void* __restrict__ bias, int bias_f32,
                                                        TOut* __restrict__ out, int M, int N, int K,
                                                        int ldx, int ldo) {
    constexpr int MT = BT / 16;                     // micro-tile edge
    constexpr int PER = BT * GT_K / 256;            // elements of each operand a thread loads per K step
    __shared__ float xs[GT_K][BT + 4];
    __shared__ float ws[GT_K][BT + 4];
    const int m0 = blockIdx.y * BT, n0 = blockIdx.x * BT;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    // loaders: BT rows x 16 k per operand, PER consecutive k per thread
    const int lrow = threadIdx.x / (GT_K / PER);
    const int lk = (threadIdx.x % (GT_K / PER)) * PER;
    float acc[MT][MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GT_K) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int k = k0 + lk + i;
            const int m = m0 + lrow, n = n0 + lrow;
            xs[lk + i][lrow] = (m < M && k < K) ? to_float(x[(size_t)m * ldx + k]) : 0.f;
            ws[lk + i][lrow] = (n < N && k < K) ? to_float(w[(size_t)n * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GT_K; ++k) {
            float a[MT], b[MT];
#pragma unroll
            for (int i = 0; i < MT; ++i) a[i] = xs[k][ty * MT + i];
#pragma unroll
            for (int j = 0; j < MT; ++j) b[j] = ws[k][tx * MT + j];
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < MT; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = m0 + ty * MT + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int n = n0 + tx * MT + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias) v += load_vec(bias, bias_f32, n);
            out[(size_t)m * ldo + n] = from_float<TOut>(v);
        }
    }
}

template <typename TIn, typename TOut>
static void launch_gemm_tile(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                             int ldx, int ldo, hipStream_t stream) {
    if (M >= 128 && N >= 128) {
        dim3 grid((N + 127) / 128, (M + 127) / 128), block(256);
        gemm_tile_kernel<TIn, TOut, 128><<<grid, block, 0, stream>>>((const TIn*)x, (const TIn*)w, bias, bias_f32, (TOut*)out, M, N, K, ldx, ldo);
    } else {
        dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
        gemm_tile_kernel<TIn, TOut, 64><<<grid, block, 0, stream>>>((const TIn*)x, (const TIn*)w, bias, bias_f32, (TOut*)out, M, N, K, ldx, ldo);
    }
}

// dtype: of x and w.  out_f32: write 32-bit results (logits) whatever the input dtype.
extern "C" int tl_gemm_general(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                               int M, int N, int K, int ldx, int ldo, int dtype, int out_f32,
                               hipStream_t stream) {
    TL_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldo >= N, "gemm: bad sizes M=%d N=%d K=%d ldx=%d ldo=%d", M, N, K, ldx, ldo);
    if (M == 0) return TL_OK;
    if (dtype == TL_DT_F32) launch_gemm_tile<float, float>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
    else if (dtype == TL_DT_BF16 && out_f32) launch_gemm_tile<bf16_t, float>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
    else if (dtype == TL_DT_BF16) launch_gemm_tile<bf16_t, bf16_t>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
    else TL_REQUIRE(false, "gemm: unknown dtype %d", dtype);
    TL_CHECK_LAUNCH("gemm_general");
    return TL_OK;
}


// =====================================================================================
// True 32-bit, few rows (M <= 16): the decode step's products of the 32-bit engine.
//
// The tile kernel above computes a 64-row tile whatever M is; with one to sixteen rows the
// product is a stream of the weight matrix and wants nothing but loads in flight.  A wave owns
// two weight rows; its lanes walk them in 16-byte pieces (lane, lane + 64, ...), multiply each
// piece with the matching piece of every x row (GV_KC columns of x at a time wait in shared
// memory) and keep one partial sum per (x row, weight row); at the end the 64 partial sums are
// added up in a fixed butterfly order.  A row's result therefore depends on neither M nor the
// other rows, as in the tile kernel, but its rounding differs from the tile kernel's (another
// order of the same sum).  Needs K % 4 == 0 and 16-byte aligned rows.
#define GV_ROWS 8
template <int MR>
__global__ __launch_bounds__(256) void gemv_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                       const void* __restrict__ bias, int bias_f32,
                                                       float* __restrict__ out, int M, int N, int K, int ldx, int ldo) {
    constexpr int KC = MR >= 8 ? 512 : 1024;       // 32 KB of x at most; at eight rows the shorter chunk keeps the kernel to 128 registers
    __shared__ float4 xs[MR][KC / 4];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n0 = blockIdx.x * GV_ROWS + wave * 2;
    const float* wa = w + (size_t)min(n0, N - 1) * K;        // rows past the end: read the last row, write nothing
    const float* wb = w + (size_t)min(n0 + 1, N - 1) * K;
    float acc[MR][2];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m][0] = acc[m][1] = 0.f;

    // A lane's pieces of its two rows are lane, lane + 64, ...: IPC of them per chunk of x.  The pieces of the next
    // chunk are requested while this chunk's are multiplied, so the stream of weights does not stop at the barriers
    // around the copy of x (with the requests made inside a chunk only, every chunk began with an empty pipe: the
    // 7B's decode step in 32-bit 9.5 -> see the measurements).  A piece beyond the row's end is fetched from the
    // row's last piece and cleared.
    constexpr int IPC = KC / 4 / 64;
    const int all = K / 4;
    float4 ra[IPC], rb[IPC];
    auto fetch = [&](int j, int c) {
        const int cc = min(c, all - 1);
        ra[j] = *(const float4*)(wa + 4 * cc);
        rb[j] = *(const float4*)(wb + 4 * cc);
    };
#pragma unroll
    for (int j = 0; j < IPC; ++j) fetch(j, lane + 64 * j);
    for (int k0 = 0; k0 < K; k0 += KC) {
        const int pieces = min(KC, K - k0) / 4;
        __syncthreads();
        for (int i = threadIdx.x; i < MR * (KC / 4); i += 256) {
            const int m = i / (KC / 4), c = i % (KC / 4);
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < M && c < pieces) v = *(const float4*)(x + (size_t)m * ldx + k0 + 4 * c);
            xs[m][c] = v;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < IPC; ++j) {
            const int c = lane + 64 * j;
            float4 a = ra[j], b = rb[j];
            if (k0 + KC < K) fetch(j, (k0 + KC) / 4 + c);
            if (c >= pieces) a = b = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const float4 xv = xs[m][c];
                acc[m][0] = fmaf(a.w, xv.w, fmaf(a.z, xv.z, fmaf(a.y, xv.y, fmaf(a.x, xv.x, acc[m][0]))));
                acc[m][1] = fmaf(b.w, xv.w, fmaf(b.z, xv.z, fmaf(b.y, xv.y, fmaf(b.x, xv.x, acc[m][1]))));
            }
            // (one piece's reads of x at a time: moved up across the pieces they take the kernel from 112 to 192
            // registers at eight rows, and half the waves fit a compute unit)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int r = 0; r < 2; ++r) acc[m][r] = wave_sum(acc[m][r]);
    if (lane < 2 && n0 + lane < N) {
        const int n = n0 + lane;
        const float b = bias ? load_vec(bias, bias_f32, n) : 0.f;
#pragma unroll
        for (int m = 0; m < MR; ++m)
            if (m < M) out[(size_t)m * ldo + n] = (lane ? acc[m][1] : acc[m][0]) + b;
    }
}

// The same on the matrix cores, 2 to 16 rows: v_mfma_f32_16x16x4_f32 multiplies and adds in true 32-bit (as
// v_mfma_f32_32x32x2_f32 below), and a step of several rows costs the stream of weights and little else, where the
// kernel above spends a multiply-add per row and weight (the dispatch takes this kernel from 9 rows on).  A work-group of eight waves owns 16 weight rows; chunks of GM_KC columns of x wait in shared
// memory (rows beyond M as zeros); within a chunk the waves take its pieces of 16 columns in turn.  A lane fetches
// four neighbouring k of its weight row and of its x row at once: lane group g = lane / 16 takes k = 4 g .. 4 g + 3
// of the piece, so instruction e of a piece multiplies k = 4 g + e of the four groups: which k meet in one instruction
// is free as long as both operands agree.  The pieces of the next chunk are requested while this chunk's are
// multiplied.  Each wave's sum over its pieces runs in one fixed order and the eight partial tiles are added in wave
// order, whatever M is: a row's result does not depend on the batch (it differs from the other 32-bit kernels' by
// rounding).  Needs K % 4 == 0 and 16-byte aligned rows.
typedef float gm_f32x4_t __attribute__((ext_vector_type(4)));
#define GM_WAVES 8
#define GM_KC 512                        // columns of x in shared memory at a time: 16 rows x 512 x 4 bytes = 32 KB
#define GM_LD (GM_KC + 4)                // floats between rows of x: 16-byte reads of 16 rows fall on all banks
__global__ __launch_bounds__(GM_WAVES * 64) void gemv_f32_mfma_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                      const void* __restrict__ bias, int bias_f32,
                                                                      float* __restrict__ out, int M, int N, int K, int ldx, int ldo) {
    __shared__ __attribute__((aligned(16))) float xs[16 * GM_LD];
    __shared__ __attribute__((aligned(16))) float red[GM_WAVES * 256];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const float* wrow = w + (size_t)min(n0 + li, N - 1) * K;       // rows past the end: the last row again, never stored
    constexpr int PPW = GM_KC / 16 / GM_WAVES;                     // pieces of 16 columns a wave takes of a chunk
    gm_f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
    float4 ring[PPW];
    // piece q of the chunk at k0 that is this wave's: columns k0 + 16 (wave + q GM_WAVES) + 4 lg .. + 3; beyond K the
    // row's last whole four are fetched and cleared
    auto fetch = [&](int q, int k0) {
        const int k = k0 + 16 * (wave + q * GM_WAVES) + 4 * lg;
        ring[q] = *(const float4*)(wrow + min(k, K - 4));
        if (k >= K) ring[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    };
#pragma unroll
    for (int q = 0; q < PPW; ++q) fetch(q, 0);
    for (int k0 = 0; k0 < K; k0 += GM_KC) {
        const int cols = min(GM_KC, K - k0);
        __syncthreads();                                           // the chunk before is read
        for (int i = tid; i < 16 * (GM_KC / 4); i += GM_WAVES * 64) {
            const int m = i / (GM_KC / 4), c = i % (GM_KC / 4);
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < M && 4 * c < cols) v = *(const float4*)(x + (size_t)m * ldx + k0 + 4 * c);
            *(float4*)(&xs[m * GM_LD + 4 * c]) = v;
        }
        __syncthreads();
#pragma unroll
        for (int q = 0; q < PPW; ++q) {
            const float4 a = ring[q];
            if (k0 + GM_KC < K) fetch(q, k0 + GM_KC);
            const float4 b = *(const float4*)(&xs[li * GM_LD + 16 * (wave + q * GM_WAVES) + 4 * lg]);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b.w, acc, 0, 0, 0);
        }
    }
    // a lane holds weight rows i = 4 (lane / 16) + v and x row j = lane % 16 of its wave's partial tile
    *(gm_f32x4_t*)(&red[(wave * 64 + lane) * 4]) = acc;
    __syncthreads();
    if (wave == 0) {
        gm_f32x4_t sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int wv = 0; wv < GM_WAVES; ++wv) sum += *(const gm_f32x4_t*)(&red[(wv * 64 + lane) * 4]);
        const int m = li;
        if (m < M) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int n = n0 + 4 * lg + v;
                if (n < N) out[(size_t)m * ldo + n] = sum[v] + (bias ? load_vec(bias, bias_f32, n) : 0.f);
            }
        }
    }
}

static bool gemv_f32_fits(const void* x, const void* w, int M, int K, int ldx) {
    return M <= 16 && K % 4 == 0 && ldx % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
}

// mfma: 0 the multiply-add kernel, 1 the matrix-core kernel, -1 the one that is faster for M.  Measured on the four
// products of a 7B layer (us, multiply-adds / matrix cores): 1 row 174 / 237, 4 rows 216 / 241, 8 rows 274 / 265,
// 16 rows 425 / 300: the matrix-core kernel's time hardly grows with the rows, but its work-groups of 16 weight rows
// are too few on the narrow matrices (224 for 3584 rows) to stream as fast as the other's 448 of 8.
static void launch_gemv_f32(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                            int ldx, int ldo, hipStream_t stream, int mfma = -1) {
    if (mfma == 1 || (mfma < 0 && M > 8)) {
        gemv_f32_mfma_kernel<<<dim3((N + 15) / 16), dim3(GM_WAVES * 64), 0, stream>>>((const float*)x, (const float*)w, bias, bias_f32,
                                                                                     (float*)out, M, N, K, ldx, ldo);
        return;
    }
    dim3 grid((N + GV_ROWS - 1) / GV_ROWS), block(256);
#define GV_LAUNCH(MR) gemv_f32_kernel<MR><<<grid, block, 0, stream>>>((const float*)x, (const float*)w, bias, bias_f32, (float*)out, M, N, K, ldx, ldo)
    if (M <= 1) GV_LAUNCH(1);
    else if (M <= 2) GV_LAUNCH(2);
    else if (M <= 4) GV_LAUNCH(4);
    else if (M <= 8) GV_LAUNCH(8);
    else GV_LAUNCH(16);
#undef GV_LAUNCH
}

// =====================================================================================
// True 32-bit on the matrix cores, more than 16 rows: the prompt steps of the 32-bit engine.
//
// v_mfma_f32_32x32x2_f32 multiplies 32-bit operands and adds in 32-bit: it is no reduced-precision mode
// (nothing is rounded to a shorter format on the way), and it runs at four times the rate of the
// v_fma_f32 tile kernel above.  A work-group of four waves owns a tile of BM x 128 outputs (BM = 64 or
// 128), a wave 32 FMB x 64 of them; slabs of 16 columns of both operands go through registers into shared
// memory (two buffers, one barrier per slab).  A lane reads four neighbouring k of its row at once; lanes
// 0-31 take k = 8c .. 8c+3 and lanes 32-63 k = 8c+4 .. 8c+7 of a chunk of eight, so instruction e of a chunk
// multiplies k = 8c + e and 8c + 4 + e: which k meet in one instruction is free as long as both operands
// agree.  The sum of an output element runs in that one fixed order whatever M is and wherever the element
// lies in its tile, so a row's result does not depend on the batch; it differs from the other 32-bit
// kernels' by rounding (another order of the same sum).  Needs K % 4 == 0 and 16-byte aligned rows.
typedef float gf_f32x16_t __attribute__((ext_vector_type(16)));
#define GF_BN 128
#define GF_TK 16
#define GF_LD (GF_TK + 4)          // floats between rows in shared memory: 16-byte reads of 16 rows fall on all banks
template <int FMB>
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            const void* __restrict__ bias, int bias_f32,
                                                            float* __restrict__ out, int M, int N, int K, int ldx, int ldo) {
    constexpr int BM = 64 * FMB;
    constexpr int XL = BM * 4 / 256;                       // 16-byte pieces of x a thread moves per slab (1 or 2)
    __shared__ __attribute__((aligned(16))) float xs[2][BM * GF_LD];
    __shared__ __attribute__((aligned(16))) float ws[2][GF_BN * GF_LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lr = lane & 31, lh = lane >> 5;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * GF_BN;

    gf_f32x16_t acc[2][FMB];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < FMB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // piece p of a slab: row p / 4, columns 4 (p % 4) .. + 4; rows past the end read the last row (never stored),
    // columns past K read the last whole piece and count as zero
    float4 gx[XL], gw[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int p = tid + 256 * i, k = k0 + 4 * (p & 3);
            gx[i] = *(const float4*)(x + (size_t)min(m0 + (p >> 2), M - 1) * ldx + min(k, K - 4));
            if (k >= K) gx[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int p = tid + 256 * i, k = k0 + 4 * (p & 3);
            gw[i] = *(const float4*)(w + (size_t)min(n0 + (p >> 2), N - 1) * K + min(k, K - 4));
            if (k >= K) gw[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto park = [&](int buf) {
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int p = tid + 256 * i;
            *(float4*)(&xs[buf][(p >> 2) * GF_LD + 4 * (p & 3)]) = gx[i];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int p = tid + 256 * i;
            *(float4*)(&ws[buf][(p >> 2) * GF_LD + 4 * (p & 3)]) = gw[i];
        }
    };
    fetch(0);
    park(0);
    __syncthreads();
    const int slabs = (K + GF_TK - 1) / GF_TK;
    for (int s = 0; s < slabs; ++s) {
        if (s + 1 < slabs) fetch((s + 1) * GF_TK);          // on their way while this slab is multiplied
        const float* xb = xs[s & 1];
        const float* wb = ws[s & 1];
#pragma unroll
        for (int c = 0; c < GF_TK / 8; ++c) {
            float4 a[2], b[FMB];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = *(const float4*)(wb + (wn * 64 + i * 32 + lr) * GF_LD + 8 * c + 4 * lh);
#pragma unroll
            for (int j = 0; j < FMB; ++j) b[j] = *(const float4*)(xb + (wm * 32 * FMB + j * 32 + lr) * GF_LD + 8 * c + 4 * lh);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < FMB; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].x, b[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].y, b[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].z, b[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i].w, b[j].w, acc[i][j], 0, 0, 0);
                }
        }
        if (s + 1 < slabs) park((s + 1) & 1);               // everyone left that buffer before the last barrier
        __syncthreads();
    }
    // weight block times x block: a lane holds row m = lane % 32 of x and the output columns
    // n = 8 (v / 4) + 4 (lane / 32) + v % 4 of a 32 x 32 block, four neighbours at a time
    const bool quads = N % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)out % 16) == 0;
#pragma unroll
    for (int j = 0; j < FMB; ++j) {
        const int m = m0 + wm * 32 * FMB + j * 32 + lr;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * 64 + i * 32 + 8 * g + 4 * lh;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * g + e] + ((bias && n + e < N) ? load_vec(bias, bias_f32, n + e) : 0.f);
                if (quads) {
                    if (n < N) *(float4*)(out + (size_t)m * ldo + n) = make_float4(v[0], v[1], v[2], v[3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < N) out[(size_t)m * ldo + n + e] = v[e];
                }
            }
    }
}

static bool gemm_f32_mfma_fits(const void* x, const void* w, int M, int K, int ldx) {
    return M > 16 && K >= 4 && K % 4 == 0 && ldx % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
}

static void launch_gemm_f32_mfma(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                                 int ldx, int ldo, hipStream_t stream) {
    // tiles of 64 rows where those of 128 would leave most compute units without one
    const long tiles128 = (long)((M + 127) / 128) * ((N + GF_BN - 1) / GF_BN);
    if (M <= 64 || tiles128 < 256) {
        dim3 grid((N + GF_BN - 1) / GF_BN, (M + 63) / 64);
        gemm_f32_mfma_kernel<1><<<grid, dim3(256), 0, stream>>>((const float*)x, (const float*)w, bias, bias_f32, (float*)out, M, N, K, ldx, ldo);
    } else {
        dim3 grid((N + GF_BN - 1) / GF_BN, (M + 127) / 128);
        gemm_f32_mfma_kernel<2><<<grid, dim3(256), 0, stream>>>((const float*)x, (const float*)w, bias, bias_f32, (float*)out, M, N, K, ldx, ldo);
    }
}

// One named kernel of the 32-bit products (for tests and tuning): 0 the general tile kernel (v_fma_f32), 1 the matrix-core
// tile kernel, 2 and 3 the kernels for up to 16 rows on multiply-adds and on the matrix cores.
extern "C" int tl_gemm_f32_variant(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                                   int M, int N, int K, int ldx, int ldo, int matrix_cores, hipStream_t stream) {
    TL_REQUIRE(M > 0 && N > 0 && K > 0 && ldx >= K && ldo >= N, "gemm_f32: bad sizes M=%d N=%d K=%d ldx=%d ldo=%d", M, N, K, ldx, ldo);
    if (matrix_cores == 2 || matrix_cores == 3) {      // the two kernels for up to 16 rows: 2 multiply-adds, 3 matrix cores
        TL_REQUIRE(gemv_f32_fits(x, w, M, K, ldx), "gemm_f32: the few-rows kernels need M <= 16, K %% 4 == 0 and 16-byte aligned rows");
        launch_gemv_f32(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream, matrix_cores - 2);
    } else if (matrix_cores) {
        TL_REQUIRE(gemm_f32_mfma_fits(x, w, 17, K, ldx), "gemm_f32: the matrix-core kernel needs K %% 4 == 0 and 16-byte aligned rows");
        launch_gemm_f32_mfma(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
    } else {
        launch_gemm_tile<float, float>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
    }
    TL_CHECK_LAUNCH("gemm_f32");
    return TL_OK;
}

// =====================================================================================
// bfloat16 on the matrix cores, few rows (M <= 64): the decode step's products.
//
// Such a product is a stream of the weight matrix through the chip once; the kernel is
// built so that nothing but HBM limits it.  out^T tile = W tile * x^T on
// v_mfma_f32_16x16x32_bf16: the A operand is 16 rows of W, the B operand 16 rows of x, both
// read straight from memory as 16-byte pieces of a K-contiguous row (no shared-memory
// staging, no barrier in the loop).  A wave owns R strips of 16 weight rows and MT tiles of
// 16 activation rows and walks K in steps of 64: lane group g = lane / 16 reads the 32
// contiguous bytes k = 64 s + 16 g .. + 16 of its row, so the four groups of a row consume
// one full 128-byte line; the two 16-byte halves feed two MFMAs (how k is dealt to lanes is
// free as long as A and B agree).  The KS waves of a work-group take the steps s = wave,
// wave + KS, ... and add their partial tiles through shared memory in a fixed order, so
// the result is deterministic.  One row of x is as good as free (the lanes of a wave that read the
// same address share the fetch); with more rows x costs M / 16 of the weight traffic again, so it is
// copied into shared memory (XL) by no more work-groups than the compute units hold at once, each
// of which then walks a run of outputs of its own, strip after strip, and requests the first
// steps of its next strip before it adds up the sums of this one (measured at M = 8, 7B sizes:
// gate/up 57 -> 51 us, LM head 207 -> 189 us).
// Needs K % 8 == 0 and 16-byte aligned rows; other shapes go to the general kernel.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define SK_KOFF(lg) (16 * (lg))     // a lane reads 32 contiguous bytes per step (other splits measured the same)
#define SK_SECOND 8
#define SK_LOAD(p) (*(const uint4*)(p))

union Frag16 {          // 16 bytes: eight bfloat16 as the MFMA wants them, or one 128-bit load
    uint4 u;
    bf16x8_t v;
};

__device__ __forceinline__ void lds_barrier() {
    // waits for this wave's shared-memory traffic only: weight fetches stay in flight across it
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Register sets of weights a wave of the skinny kernel keeps in flight: as many K steps as fit
// beside the accumulators (a step takes 8 registers per strip and 8 per tile of activation rows).
template <int R, int MT, int KS>
constexpr int skinny_depth() {
    const int per_step = 8 * R + 8 * MT;
    const int budget = KS >= 16 ? 64 : 128;       // 1024 threads leave 128 registers a lane
    const int d = budget / per_step;
    return d < 2 ? 2 : (d > 8 ? 8 : d);
}

__device__ __forceinline__ float silu_mul(float g, float u) { return g / (1.f + expf(-g)) * u; }

// SW (gate/up product with the SwiGLU gate applied to the accumulators): w holds blocks of 64
// rows, 32 gate rows followed by the 32 up rows of the same columns; a work-group's strip is up to 16
// outputs, whose gate rows half of its waves walk and whose up rows the other half (R == 1: each
// wave streams one strip of 16 rows, which is what reaches the memory's rate; four strips per
// wave, as an earlier version had, stayed at 56-58 us on the 7B's matrix where this takes 50-53);
// out has N / 2 columns.
// XL (x through shared memory): with more than one activation row the 16 lanes of a group read
// 16 different rows of x, which no longer fit the L1 cache once M * K * 2 bytes exceed it, and
// every operand load of x becomes a trip to L2 that competes with the weight stream (measured:
// 5.6 TB/s at M = 1, 4.6 at M = 8, 3.7 at M = 16 without it).  With XL the work-group copies
// its M rows of x into shared memory once, coalesced, and reads the operands from there.
// D: how many K steps of weights a wave keeps in flight (a ring of D register sets).  Short
// rows (a few steps per wave) want them all in flight at once, or every step costs a trip to memory.
// RP (the fused query/key/value projection of a decode step, R == 1 and MT == 1): the epilogue rotates
// the query and key heads by the token's position and puts keys and values into their pages, so no
// kernel of its own has to.  The projection's rows are in the pair layout: the two elements that
// frequency j turns are the neighbouring output columns 2j and 2j + 1 of a head, both in one lane.
struct RopeArgs {
    const int* positions;      // [M]
    const float* inv_freq;     // [head_dim / 2]
    const int* token_req;      // [M] request of each row (null: no cache write)
    const int* block_table;    // [requests, bt_stride]
    bf16_t* k_plane;           // [pages, kv_heads, page, head_dim]
    bf16_t* v_plane;           // [pages, kv_heads, head_dim, page]
    int bt_stride, page, q_heads, kv_heads, head_dim;
};

// Eight neighbouring elements as floats, from float or bfloat16 memory and back.
__device__ __forceinline__ void load8(const float* p, float* v) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float* v) {
    const uint4 t = *(const uint4*)p;
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    v[4] = __uint_as_float(t.z << 16); v[5] = __uint_as_float(t.z & 0xffff0000u);
    v[6] = __uint_as_float(t.w << 16); v[7] = __uint_as_float(t.w & 0xffff0000u);
}
__device__ __forceinline__ void store8(float* p, const float* v) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
    *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float* v) {
    uint4 t;
    t.x = (uint32_t)from_float<bf16_t>(v[0]).bits | ((uint32_t)from_float<bf16_t>(v[1]).bits << 16);
    t.y = (uint32_t)from_float<bf16_t>(v[2]).bits | ((uint32_t)from_float<bf16_t>(v[3]).bits << 16);
    t.z = (uint32_t)from_float<bf16_t>(v[4]).bits | ((uint32_t)from_float<bf16_t>(v[5]).bits << 16);
    t.w = (uint32_t)from_float<bf16_t>(v[6]).bits | ((uint32_t)from_float<bf16_t>(v[7]).bits << 16);
    *(uint4*)p = t;
}

// r += the N slabs' eight elements at src, src + stride, ...: all requested, then added in their order.
template <int N>
__device__ __forceinline__ void add_slabs8(const float* src, size_t stride, float (&r)[8]) {
    float p[N][8];
#pragma unroll
    for (int u = 0; u < N; ++u) load8(src + u * stride, p[u]);
#pragma unroll
    for (int u = 0; u < N; ++u)
#pragma unroll
        for (int v = 0; v < 8; ++v) r[v] += p[u][v];
}

// NF (one row, with XL): x is not read but made here, as the norm of the residual stream would make it:
// r = residual + pending (bfloat16, or float slabs of partial sums), x = r * rsqrt(mean(r^2) + eps) * weight, all
// in 32-bit and rounded once; the first work-group writes r out as the new residual (to another place than it
// is read from: the others may still be reading).  Every work-group does this once for all the strips it
// walks, while its first weights are on their way; the norm's own kernel, a launch and a trip to memory with
// nothing else to do, is not run at all (7B sizes, one row: 4.6 us twice a layer).
struct NormArgs {
    const float* residual;     // [K]
    float* residual_out;       // [K]
    const void* pending;       // bfloat16 [K], or float [parts][part_stride], or null
    const void* weight;        // [K], bfloat16 or float
    size_t part_stride;
    int parts, weight_f32;
    float eps;
};

template <int R, int MT, int KS, typename TOut, bool SW = false, bool XL = false, int D = 2, bool RP = false, bool NF = false>
__global__ __launch_bounds__(KS * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                              const void* __restrict__ bias, int bias_f32,
                                                              TOut* __restrict__ out, int M, int N, int K, int ldx, int ldo,
                                                              int out_cols, int k_per_split, int rows_per_strip, int rows_per_group,
                                                              RopeArgs ra, NormArgs na) {
    static_assert(!NF || (XL && MT == 1), "the fused norm makes x in shared memory, for one row");
    static_assert(!SW || (R == 1 && KS % 2 == 0), "the fused gate deals a work-group's waves to a gate strip and its up strip");
    static_assert(!RP || (R <= 2 && MT == 1 && !SW), "the fused rotation is built for up to 16 rows of x");
    // Split K (k_per_split > 0, a multiple of 64): blockIdx.y owns the columns
    // [y * k_per_split, ...) of x and w and writes its own [M, ldo] slab of partial sums to out
    // (float, no bias); whoever reads them adds the slabs up.
    const int ldw = K;
    if (k_per_split > 0) {
        const int kb = blockIdx.y * k_per_split;
        x += kb;
        w += kb;
        out += (size_t)blockIdx.y * M * ldo;
        K = min(K - kb, k_per_split);
    }
    extern __shared__ __attribute__((aligned(16))) float skinny_lds[];
    float* red = skinny_lds;                                             // KS * R * MT * 256 floats
    bf16_t* xs = (bf16_t*)(skinny_lds + KS * R * MT * 256);             // XL: M rows of K + 8 elements
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    // The outputs (weight rows; with the fused gate, SW, pairs of a gate row and an up row) are dealt to the
    // work-groups in runs of rows_per_group, and a work-group walks its run in strips of rows_per_strip, up to
    // 16 R (0: exactly that; rows_per_group 0: one strip).  A compute unit draws its weights at a rate of its
    // own, about 26 GB/s whatever it shares the chip with, so a product takes as long as its busiest unit: 257
    // strips of 16 rows take as long as 512 (11.2 against 7.9 us for 256, at 3584 columns), and equal shares for
    // all work-groups are worth more than full blocks of 16 rows.  Lanes beyond a strip's last row fetch copies
    // of it and store nothing.  Only with x in shared memory (XL) does a work-group walk more than one strip:
    // x is copied (or made, NF) once for all of them, and the first fetches of the next strip are on their way
    // while the sums of this one are added up.
    // With the fused gate the first KS / 2 waves walk K for the gate rows of the strip's outputs, the others
    // for the up rows of the same outputs (the interleaved matrix holds blocks of 32 gate rows followed by
    // their 32 up rows), and the sums of both meet in shared memory.
    constexpr int KW = SW ? KS / 2 : KS;       // waves along K per strip
    const int kwave = SW ? wave % KW : wave;
    const int total = SW ? out_cols : N;
    const int rps = rows_per_strip > 0 ? rows_per_strip : 16 * R;
    const int run_begin = blockIdx.x * ((XL && rows_per_group > 0) ? rows_per_group : rps);
    const int run_end = min(total, run_begin + ((XL && rows_per_group > 0) ? rows_per_group : rps));
    auto strip_begin = [&](int i) { return run_begin + i * rps; };
    auto strip_end = [&](int i) { return min(run_begin + i * rps + rps, run_end); };
    auto lane_row = [&](int i, int r) {        // the weight row this lane fetches for block r of strip i
        const int o = min(strip_begin(i) + r * 16 + li, strip_end(i) - 1);
        return SW ? (o >> 5) * 64 + (wave / KW) * 32 + (o & 31) : o;
    };
    int strip = 0;
    int rp_pos = 0, rp_page = 0;               // RP: this lane's row (li), fetched now, used in the epilogue
    if (RP) {
        const int row = min(li, M - 1);
        rp_pos = ra.positions[row];
        if (ra.k_plane) rp_page = ra.block_table[(size_t)ra.token_req[row] * ra.bt_stride + rp_pos / ra.page];
    }

    const bf16_t* wrow[R];
    const bf16_t* xrow[MT];
    int xoff[MT];
#pragma unroll
    for (int r = 0; r < R; ++r) wrow[r] = w + (size_t)lane_row(strip, r) * ldw;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        xrow[t] = x + (size_t)min(t * 16 + li, M - 1) * ldx;
        xoff[t] = min(t * 16 + li, M - 1) * (K + 8);
    }
#define SK_LOADB(t, k) (XL ? *(const uint4*)(&xs[xoff[t] + (k)]) : *(const uint4*)(xrow[t] + (k)))

    f32x4_t acc[R][MT];
    const int full = K / 64;                   // steps that lie wholly inside K
    // this wave's steps are s = kwave + i * KW, i = 0 .. mine - 1; slot d of the ring holds step i = d (mod D)
    const int mine = full > kwave ? (full - kwave + KW - 1) / KW : 0;
    Frag16 wa0[D][R], wa1[D][R], wb0[D][MT], wb1[D][MT];
#define SK_ISSUE(d, i)                                                                              \
    {                                                                                               \
        const int k_ = 64 * (kwave + (i) * KW) + SK_KOFF(lg);                                       \
        _Pragma("unroll") for (int r = 0; r < R; ++r) {                                             \
            wa0[d][r].u = SK_LOAD(wrow[r] + k_);                                                    \
            wa1[d][r].u = SK_LOAD(wrow[r] + k_ + SK_SECOND);                                        \
        }                                                                                           \
        if (!XL) {                                                                                  \
            _Pragma("unroll") for (int t = 0; t < MT; ++t) {                                        \
                wb0[d][t].u = SK_LOAD(xrow[t] + k_);                                                \
                wb1[d][t].u = SK_LOAD(xrow[t] + k_ + SK_SECOND);                                    \
            }                                                                                       \
        }                                                                                           \
    }
#pragma unroll
    for (int d = 0; d < D; ++d)
        if (d < mine) SK_ISSUE(d, d)
    if (NF) {                                  // the weights are on their way while x is made
        // a thread owns up to two pieces of eight elements (the host checked K <= 16 * threads)
        const int pieces = K / 8;
        float r[2][8];
        float ss = 0.f;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int i = min((int)threadIdx.x + c * KS * 64, pieces - 1) * 8;
            load8(na.residual + i, r[c]);
            if (na.pending && na.parts == 0) {
                float p[8];
                load8((const bf16_t*)na.pending + i, p);
#pragma unroll
                for (int v = 0; v < 8; ++v) r[c][v] += p[v];
            }
            const float* slab = (const float*)na.pending + i;
            if constexpr (RP) {
                // The query/key/value projection follows the down projection, whose K is split many ways: four slabs
                // at a time, all requested before the first is added, in their order (one after the other, the eight
                // slabs of the 7B's down projection were eight trips to memory before the first weight was used); the
                // last two or three are a group as well.
                int q = 0;
                for (; q + 4 <= na.parts; q += 4) add_slabs8<4>(slab + q * na.part_stride, na.part_stride, r[c]);
                if (na.parts - q == 3) add_slabs8<3>(slab + q * na.part_stride, na.part_stride, r[c]);
                else if (na.parts - q == 2) add_slabs8<2>(slab + q * na.part_stride, na.part_stride, r[c]);
                else if (na.parts - q == 1) add_slabs8<1>(slab + q * na.part_stride, na.part_stride, r[c]);
            } else {
                // (the fused gate follows the output projection, one slab or few: the registers of a group would cost
                // its work-groups of sixteen waves the second one on a compute unit)
                for (int q = 0; q < na.parts; ++q) {
                    float p[8];
                    load8(slab + q * na.part_stride, p);
#pragma unroll
                    for (int v = 0; v < 8; ++v) r[c][v] += p[v];
                }
            }
            if ((int)threadIdx.x + c * KS * 64 < pieces) {
#pragma unroll
                for (int v = 0; v < 8; ++v) ss += r[c][v] * r[c][v];
            }
        }
        ss = wave_sum(ss);
        float* sums = red;                            // free until the first strip's sums
        if (lane == 0) sums[wave] = ss;
        lds_barrier();
        float total = 0.f;
        for (int wv = 0; wv < KS; ++wv) total += sums[wv];
        const float inv = rsqrtf(total / (float)K + na.eps);
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int pc = (int)threadIdx.x + c * KS * 64;
            if (pc < pieces) {
                float g[8];
                if (na.weight_f32) load8((const float*)na.weight + pc * 8, g);
                else load8((const bf16_t*)na.weight + pc * 8, g);
                float o[8];
#pragma unroll
                for (int v = 0; v < 8; ++v) o[v] = r[c][v] * inv * g[v];
                store8(xs + pc * 8, o);
                if (blockIdx.x == 0 && blockIdx.y == 0) {
                    store8(na.residual_out + pc * 8, r[c]);
                }
            }
        }
        lds_barrier();
    } else if (XL) {                           // the weights are on their way while x is copied
        const int pieces = K / 8;                     // 16-byte pieces per row
        for (int i = threadIdx.x; i < M * pieces; i += KS * 64) {
            const int row = i / pieces, pc = i % pieces;
            *(uint4*)(&xs[row * (K + 8) + pc * 8]) = *(const uint4*)(x + (size_t)row * ldx + pc * 8);
        }
        lds_barrier();
    }
    while (true) {
        const int n0 = strip_begin(strip);     // first output column of the strip
        const int n_end = strip_end(strip);    // ... and the one after its last
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[r][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        for (int i = 0; i < mine; i += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                if (i + d < mine) {
                    if (XL) {
                        const int k = 64 * (kwave + (i + d) * KW) + SK_KOFF(lg);
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            wb0[d][t].u = *(const uint4*)(&xs[xoff[t] + k]);
                            wb1[d][t].u = *(const uint4*)(&xs[xoff[t] + k + SK_SECOND]);
                        }
                    }
#pragma unroll
                    for (int r = 0; r < R; ++r)
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa0[d][r].v, wb0[d][t].v, acc[r][t], 0, 0, 0);
                            acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa1[d][r].v, wb1[d][t].v, acc[r][t], 0, 0, 0);
                        }
                    if (i + d + D < mine) SK_ISSUE(d, i + d + D)
                }
            }
        }
        // the tail step (K % 64 != 0) belongs to the wave whose turn it is; pieces beyond K count as zero
        if ((K & 63) && (full % KW) == kwave) {
            Frag16 a0[R], a1[R], b0[MT], b1[MT];
            const int k = 64 * full + SK_KOFF(lg);
            const bool v0 = k + 8 <= K, v1 = k + SK_SECOND + 8 <= K;
            // (fetched from a clamped address and cleared afterwards: a fetch under a condition makes the
            // compiler route it through scratch memory, which every launch of the kernel then sets up)
            const int k0 = min(k, K - 8), k1 = min(k + SK_SECOND, K - 8);
            auto keep = [](uint4 v, bool ok) {
                v.x = ok ? v.x : 0u;
                v.y = ok ? v.y : 0u;
                v.z = ok ? v.z : 0u;
                v.w = ok ? v.w : 0u;
                return v;
            };
#pragma unroll
            for (int r = 0; r < R; ++r) {
                a0[r].u = keep(*(const uint4*)(wrow[r] + k0), v0);
                a1[r].u = keep(*(const uint4*)(wrow[r] + k1), v1);
            }
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                b0[t].u = keep(SK_LOADB(t, k0), v0);
                b1[t].u = keep(SK_LOADB(t, k1), v1);
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[r].v, b0[t].v, acc[r][t], 0, 0, 0);
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1[r].v, b1[t].v, acc[r][t], 0, 0, 0);
                }
        }
        const bool more = XL && strip_begin(strip + 1) < run_end;   // without the copy of x: one strip per work-group
        if (more) {                            // the next strip's first steps, before this strip's sums
#pragma unroll
            for (int r = 0; r < R; ++r) wrow[r] = w + (size_t)lane_row(strip + 1, r) * ldw;
#pragma unroll
            for (int d = 0; d < D; ++d)
                if (d < mine) SK_ISSUE(d, d)
        }

        // D[i][j]: lane holds i = 4 * (lane / 16) + v (weight row), j = lane % 16 (activation row)
        if (KS > 1) {
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    float* dst = red + ((size_t)(wave * R * MT + r * MT + t) * 64 + lane) * 4;
                    *(f32x4_t*)dst = acc[r][t];
                }
            lds_barrier();
        }
        if (SW) {
            for (int t = wave; t < MT; t += KS) {
                f32x4_t gs = f32x4_t{0.f, 0.f, 0.f, 0.f}, us = gs;
#pragma unroll
                for (int wv = 0; wv < KW; ++wv) {
                    gs += *(const f32x4_t*)(red + ((size_t)(wv * MT + t) * 64 + lane) * 4);
                    us += *(const f32x4_t*)(red + ((size_t)((KW + wv) * MT + t) * 64 + lane) * 4);
                }
                const int m = t * 16 + li;
                const int col = n0 + 4 * lg;
                if (m < M) {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (col + v < n_end) out[(size_t)m * ldo + col + v] = from_float<TOut>(silu_mul(gs[v], us[v]));
                }
            }
        } else {
            for (int tile = wave; tile < R * MT; tile += KS) {
                const int r = tile / MT, t = tile % MT;
                f32x4_t sum;
                if (KS > 1) {
                    sum = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int wv = 0; wv < KS; ++wv) sum += *(const f32x4_t*)(red + ((size_t)(wv * R * MT + tile) * 64 + lane) * 4);
                } else {
                    sum = acc[0][0];
#pragma unroll
                    for (int rr = 0; rr < R; ++rr)
#pragma unroll
                        for (int tt = 0; tt < MT; ++tt)
                            if (rr == r && tt == t) sum = acc[rr][tt];
                }
                const int m = t * 16 + li;
                const int n = n0 + r * 16 + 4 * lg;
                if (RP) {
                    // two pairs of neighbouring columns per lane (pair layout: one frequency turns a pair); a strip
                    // of a number of rows that is no multiple of four may end between them
                    if (m >= M) continue;
#pragma unroll
                    for (int pr = 0; pr < 2; ++pr) {
                        const int np = n + 2 * pr;
                        if (np + 1 >= n_end) continue;                 // strips hold an even number of rows
                        float y1 = sum[2 * pr] + (bias ? load_vec(bias, bias_f32, np) : 0.f);
                        float y2 = sum[2 * pr + 1] + (bias ? load_vec(bias, bias_f32, np + 1) : 0.f);
                        const int head = np / ra.head_dim, dd = np - head * ra.head_dim;
                        if (head < ra.q_heads + ra.kv_heads) {
                            const float angle = (float)rp_pos * ra.inv_freq[dd / 2];
                            const float c = cosf(angle), sn = sinf(angle);
                            const float t1 = y1 * c - y2 * sn;
                            const float t2 = y2 * c + y1 * sn;
                            y1 = t1;
                            y2 = t2;
                        }
                        const uint16_t e1 = from_float<bf16_t>(y1).bits, e2 = from_float<bf16_t>(y2).bits;
                        const uint32_t both = (uint32_t)e1 | ((uint32_t)e2 << 16);
                        if (head < ra.q_heads || !ra.k_plane) {
                            *(uint32_t*)((bf16_t*)out + (size_t)m * ldo + np) = both;
                        } else if (rp_page != 0) {     // page 0 is the sentinel (a padding row's): never written
                            const int kvh = (head - ra.q_heads) % ra.kv_heads, off = rp_pos % ra.page;
                            const size_t base = ((size_t)rp_page * ra.kv_heads + kvh) * ra.page * ra.head_dim;
                            if (head < ra.q_heads + ra.kv_heads) {
                                *(uint32_t*)(ra.k_plane + base + (size_t)off * ra.head_dim + dd) = both;
                            } else {
                                ra.v_plane[base + (size_t)dd * ra.page + off].bits = e1;
                                ra.v_plane[base + (size_t)(dd + 1) * ra.page + off].bits = e2;
                            }
                        }
                    }
                    continue;
                }
                if (m < M) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        if (n + v < n_end) {
                            float val = sum[v];
                            if (bias) val += load_vec(bias, bias_f32, n + v);
                            out[(size_t)m * ldo + n + v] = from_float<TOut>(val);
                        }
                    }
                }
            }
        }
        if (!more) break;
        ++strip;
        if (KS > 1) lds_barrier();             // the sums are read until here; the next strip's overwrite them
    }
#undef SK_ISSUE
}

// Shared memory beyond 64 KB has to be allowed per kernel, once per process.
template <typename Kernel>
static hipError_t allow_lds(Kernel kernel, size_t bytes) {
    if (bytes <= 65536) return hipSuccess;
    return hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

#define SKINNY_XL_MAX_BYTES (60 * 1024)      // x may take this much shared memory: with the reduction buffer two
                                             // work-groups still fit the 160 KB of a compute unit

// How the outputs of a product are dealt out: work-groups, the outputs of each (its run) and of a strip.
struct StripPlan {
    int groups, per_group, per_strip;
};

// Equal runs for up to `most` work-groups, each walked in equal strips of at most `cap` outputs (a multiple of
// 16); `even` keeps both numbers even (the fused rotation turns pairs of neighbouring outputs).
static StripPlan plan_strips(int total, int most, int cap, bool even) {
    StripPlan p;
    p.per_group = (total + most - 1) / most;
    if (p.per_group < 4) p.per_group = 4;                     // a strip of fewer rows wastes most of its fetches
    if (even) p.per_group += p.per_group & 1;
    const int count = (p.per_group + cap - 1) / cap;
    p.per_strip = (p.per_group + count - 1) / count;
    if (even) p.per_strip += p.per_strip & 1;
    p.groups = (total + p.per_group - 1) / p.per_group;
    return p;
}

// rows_per_strip > 0: one strip of that many outputs per work-group, whatever else holds.
template <int R, int MT, int KS, typename TOut, bool SW, int D>
static void launch_skinny_d(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                            int ldx, int ldo, int out_cols, hipStream_t stream, int rows_per_strip = 0) {
    const int total = SW ? out_cols : N;
    const int rps = rows_per_strip > 0 ? rows_per_strip : 16 * R;
    dim3 grid((total + rps - 1) / rps), block(KS * 64);
    const size_t red_bytes = (size_t)KS * R * MT * 1024;
    const size_t x_bytes = (size_t)M * (K + 8) * 2;
    // More than one row of x: two work-groups per compute unit copy x into shared memory once and walk
    // their runs of outputs (each strip's own copy took longer than it saved: 87 against 64 us on the
    // fused gate/up product at M = 8 with four waves).
    if (M > 1 && red_bytes + x_bytes <= 156 * 1024) {
        auto kernel = gemm_skinny_kernel<R, MT, KS, TOut, SW, true, D>;
        static hipError_t allowed = allow_lds(kernel, 156 * 1024);
        if (allowed == hipSuccess) {
            const int most = x_bytes <= SKINNY_XL_MAX_BYTES ? 2 * TL_COMPUTE_UNITS : TL_COMPUTE_UNITS;      // a larger x leaves room for one work-group only
            StripPlan p = plan_strips(total, most, 16 * R, false);
            if (rows_per_strip > 0) p = StripPlan{(int)grid.x, rps, rps};
            kernel<<<dim3(p.groups), block, red_bytes + x_bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (TOut*)out, M, N, K, ldx, ldo,
                                                                           out_cols, 0, p.per_strip, p.per_group, RopeArgs{}, NormArgs{});
            return;
        }
    }
    gemm_skinny_kernel<R, MT, KS, TOut, SW, false, D><<<grid, block, red_bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (TOut*)out, M, N, K, ldx, ldo,
                                                                                          out_cols, 0, rps, 0, RopeArgs{}, NormArgs{});
}

// A wave with many K steps ahead of it (a long K: the down projection) keeps as many in flight as
// its registers hold; with a few steps (K of a hidden size) two are as good and start sooner
// (measured at 3584 x 18944, one row: 33 -> 28 us with eight in flight; at 4608 x 3584: 11 -> 12.6 us).
template <int R, int MT, int KS, typename TOut, bool SW>
static void launch_skinny_t(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                            int ldx, int ldo, int out_cols, hipStream_t stream, int rows_per_strip = 0) {
    constexpr int deep = skinny_depth<R, MT, KS>();
    if (deep > 2 && K / 64 / KS >= 16)
        launch_skinny_d<R, MT, KS, TOut, SW, deep>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, rows_per_strip);
    else
        launch_skinny_d<R, MT, KS, TOut, SW, 2>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, rows_per_strip);
}

template <int R, int MT, int KS>
static void launch_skinny(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                          int ldx, int ldo, int out_f32, hipStream_t stream, int rows_per_strip = 0) {
    if (out_f32) launch_skinny_t<R, MT, KS, float, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream, rows_per_strip);
    else launch_skinny_t<R, MT, KS, bf16_t, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream, rows_per_strip);
}

// Rows a strip gets so that a matrix of N rows is dealt to the compute units in equal shares, one strip to
// each (0: the plain strips of 16 R rows are as good; *blocks: how many blocks of 16 rows a strip then has, 1 or
// 2).  A compute unit draws its weights at a rate of its own, about 26 GB/s whatever shares it with, and the strips
// beyond one per unit run when the others are done, nearly alone, at the latency of every fetch: at 3584 columns 256 strips of 16 rows take 7.9 us, 257 take 11.2, 288 (the
// 7B's query/key/value matrix) 11.9 and 512 take 13.4.  The number is even (the fused rotation turns pairs).
static int balanced_rows(int N, int* blocks) {
    *blocks = 1;
    if (N < 4 * TL_COMPUTE_UNITS || N > 32 * TL_COMPUTE_UNITS) return 0;      // a few rows a unit, or more than two blocks
    if (N % (16 * TL_COMPUTE_UNITS) == 0) return 0;                               // whole blocks already come out even
    int rows = (N + TL_COMPUTE_UNITS - 1) / TL_COMPUTE_UNITS;
    rows += rows & 1;
    *blocks = rows > 16 ? 2 : 1;
    return rows;
}

template <int MT>
static void pick_skinny(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                        int ldx, int ldo, int out_f32, hipStream_t stream) {
    // Measured on MI355X at Qwen2.5-7B sizes (weights streamed from HBM, M = 8 and 64):
    // with up to 32 rows one strip of 16 weight rows per work-group is best throughout, with
    // 16 waves along K for wide matrices (gate_up, LM head: 4.7-5.0 TB/s) and 8 for narrow
    // ones (qkv, o, down); with 64 rows the x operand weighs more and several strips per wave
    // share each x load.
    const int strips = (N + 15) / 16;
    if (MT == 1) {
        int blocks = 1;
        const int rows = balanced_rows(N, &blocks);
        if (rows > 0 && blocks == 1) return launch_skinny<1, 1, 8>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream, rows);
        if (rows > 0) return launch_skinny<2, 1, 8>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream, rows);
    }
    if (MT <= 2) {
        if (strips >= 1024) launch_skinny<1, MT, 16>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
        else launch_skinny<1, MT, 8>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
    } else {
        if (strips >= 2048) launch_skinny<4, MT, 4>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
        else if (strips >= 1024) launch_skinny<2, MT, 2>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
        else launch_skinny<1, MT, 8>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
    }
}

// One named instance of the few-rows kernel, of those the dispatch below can pick (for tests and tuning);
// rows_per_strip: 0 for strips of 16 R rows, else that many (at most 16 R).
extern "C" int tl_gemm_skinny_variant(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                                      int M, int N, int K, int ldx, int ldo, int out_f32, int R, int KS, int rows_per_strip,
                                      hipStream_t stream) {
    TL_REQUIRE(M > 0 && M <= 64 && K % 8 == 0 && ldx % 8 == 0, "gemm_skinny: needs 0 < M <= 64 and K, ldx multiples of 8");
    TL_REQUIRE(rows_per_strip >= 0 && rows_per_strip <= 16 * R, "gemm_skinny: a strip of %d blocks holds up to %d rows, not %d", R, 16 * R, rows_per_strip);
    const int MT = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
#define TL_SKINNY_CASE(r, t, k) \
    if (R == r && MT == t && KS == k) { launch_skinny<r, t, k>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream, rows_per_strip); TL_CHECK_LAUNCH("gemm_skinny"); return TL_OK; }
    // the instances pick_skinny can choose
    TL_SKINNY_CASE(1, 1, 16) TL_SKINNY_CASE(1, 2, 16) TL_SKINNY_CASE(1, 1, 8) TL_SKINNY_CASE(1, 2, 8) TL_SKINNY_CASE(2, 1, 8)
    TL_SKINNY_CASE(4, 4, 4) TL_SKINNY_CASE(2, 4, 2) TL_SKINNY_CASE(1, 4, 8)
#undef TL_SKINNY_CASE
    TL_REQUIRE(false, "gemm_skinny: no instance R=%d MT=%d KS=%d", R, MT, KS);
}

// =====================================================================================
// bfloat16 on the matrix cores, many rows (prompt portions): shared-memory tiles.
//
// A work-group of four or eight waves owns a BM x BN tile of the output and walks K in slabs of TK
// (32 or 64) elements.
// A slab of x (BM rows) and of w (BN rows) is fetched from memory as 16-byte pieces into
// registers while the previous slab is being multiplied, then parked in shared memory
// (two buffers, one barrier per slab).  Rows lie 2 TK + 16 bytes apart in shared memory (16 of
// padding) so that the 16-byte operand reads of v_mfma_f32_32x32x16_bf16 do not
// collide on banks.  Waves are laid out WGM x WGN over the tile; each multiplies
// (BM / WGM) x (BN / WGN) as blocks of 32 x 32 with float accumulators.
// Needs K % 8 == 0 and 16-byte aligned rows.
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// Which tile a shape gets (measured on MI355X at Qwen2.5-7B sizes, 2048 and 512 rows):
//   * 256 x 256 with slabs of 64 (eight waves) reuses operands best (840 TFLOP/s on the
//     gate/up product) but needs over a thousand such tiles to keep 256 compute units busy;
//   * otherwise 128 x 128 with slabs of 64 (two work-groups fit a compute unit: 512 at once),
//     except when the tile count lies between 512 and 768, where slabs of 32 (three fit) avoid
//     a second, nearly empty round;
//   * up to 64 rows: 64 x 128.
enum TileChoice { TILE_64x128, TILE_128x128_K32, TILE_128x128_K64, TILE_256x256 };
static TileChoice pick_tile(int M, int N) {
    if (M <= 64) return TILE_64x128;
    const long big = (long)((M + 255) / 256) * ((N + 255) / 256);
    if (big >= 1024) return TILE_256x256;
    const long wgs = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (wgs > 512 && wgs <= 768) return TILE_128x128_K32;
    return TILE_128x128_K64;
}

template <int BM, int BN, int WGM, int WGN, typename TOut, bool SW = false, int TK = 32>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_mfma_tile_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                             const void* __restrict__ bias, int bias_f32,
                                                             TOut* __restrict__ out, int M, int N, int K, int ldx, int ldo,
                                                             int out_cols = 0) {
    static_assert(!SW || (BN / WGN) % 64 == 0, "the fused gate needs whole 64-row blocks per wave");
    constexpr int TROW = TK + 8;                         // elements between rows in shared memory (16 bytes of padding)
    constexpr int NT = 64 * WGM * WGN;                   // threads
    constexpr int WM = BM / WGM, WN = BN / WGN;          // wave tile
    constexpr int FM = WM / 32, FN = WN / 32;            // 32x32 blocks per wave
    constexpr int PIECES = (BM + BN) * (TK / 8);         // 16-byte pieces per slab
    constexpr int PPT = PIECES / NT;                     // pieces per thread
    static_assert(PIECES % NT == 0, "slab must divide over the threads");
    extern __shared__ __attribute__((aligned(16))) bf16_t lds_raw[];
    bf16_t (*lds)[(BM + BN) * TROW] = (bf16_t (*)[(BM + BN) * TROW])lds_raw;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    // Which tile this work-group owns.  Work-groups are dealt to the 8 XCDs round-robin by
    // blockIdx, and each XCD has an L2 of its own: give every XCD a contiguous range of
    // "logical" tile numbers, and number tiles so that 64 consecutive ones (what an XCD runs at
    // a time) form an 8 x 8 block of the output, so that each operand tile it fetches is used
    // by eight work-groups out of its L2.
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int lid;
    {
        const int total = gridDim.x, xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
        lid = xcd * (total / 8) + min(xcd, total % 8) + idx;
    }
    int tm, tn;
    {
        const int per_group = 8 * tiles_n;
        const int first_m = (lid / per_group) * 8;
        const int rows = min(tiles_m - first_m, 8);
        tm = first_m + (lid % per_group) % rows;
        tn = (lid % per_group) / rows;
    }
    const int m0 = tm * BM, n0 = tn * BN;

    // which pieces this thread fetches: piece p -> (row, 8-element column) of the stacked [x rows; w rows] slab
    const bf16_t* src[PPT];
    int dst[PPT];
    int kcol[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
        const int p = tid + i * NT;
        const int row = p / (TK / 8), c = p % (TK / 8);
        kcol[i] = c * 8;
        dst[i] = row * TROW + c * 8;
        if (row < BM) src[i] = x + (size_t)min(m0 + row, M - 1) * ldx + c * 8;
        else src[i] = w + (size_t)min(n0 + row - BM, N - 1) * K + c * 8;
    }

    f32x16_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int slabs = (K + TK - 1) / TK;
    uint4 stage[PPT];
#pragma unroll
    for (int i = 0; i < PPT; ++i) stage[i] = (kcol[i] + 8 <= K) ? *(const uint4*)(src[i]) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < PPT; ++i) *(uint4*)(&lds[0][dst[i]]) = stage[i];
    __syncthreads();

    const int fr = lane & 31, fk = (lane >> 5) * 8;      // operand fragment: row within block, k offset
    for (int sl = 0; sl < slabs; ++sl) {
        const int cur = sl & 1;
        if (sl + 1 < slabs) {
            const int k0 = (sl + 1) * TK;
#pragma unroll
            for (int i = 0; i < PPT; ++i)
                stage[i] = (k0 + kcol[i] + 8 <= K) ? *(const uint4*)(src[i] + k0) : make_uint4(0, 0, 0, 0);
        }
        const bf16_t* xs = &lds[cur][0];
        const bf16_t* ws = &lds[cur][BM * TROW];
#pragma unroll
        for (int kk = 0; kk < TK; kk += 16) {
            Frag16 af[FM], bfr[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) af[i].u = *(const uint4*)(xs + (wm * WM + i * 32 + fr) * TROW + kk + fk);
#pragma unroll
            for (int j = 0; j < FN; ++j) bfr[j].u = *(const uint4*)(ws + (wn * WN + j * 32 + fr) * TROW + kk + fk);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i].v, bfr[j].v, acc[i][j], 0, 0, 0);
        }
        if (sl + 1 < slabs) {
#pragma unroll
            for (int i = 0; i < PPT; ++i) *(uint4*)(&lds[cur ^ 1][dst[i]]) = stage[i];
        }
        __syncthreads();
    }

    // block result: lane holds column (lane % 32), rows 8 * (v / 4) + 4 * (lane / 32) + v % 4
    if (SW) {   // even blocks hold gate columns, the next block the up columns of the same outputs
#pragma unroll
        for (int j = 0; j + 1 < FN; j += 2) {
            const int col = (n0 + wn * WN + j * 32) / 2 + (lane & 31);
            if (col >= out_cols) continue;
#pragma unroll
            for (int i = 0; i < FM; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int m = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                    if (m < M) out[(size_t)m * ldo + col] = from_float<TOut>(silu_mul(acc[i][j][v], acc[i][j + 1][v]));
                }
            }
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < FN; ++j) {
        const int n = n0 + wn * WN + j * 32 + (lane & 31);
        if (n >= N) continue;
        const float b = bias ? load_vec(bias, bias_f32, n) : 0.f;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm * WM + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (m < M) out[(size_t)m * ldo + n] = from_float<TOut>(acc[i][j][v] + b);
            }
        }
    }
}

// Shared memory of a tile kernel: two buffers of (BM + BN) rows of TK + 8 elements.

template <int BM, int BN, int WGM, int WGN, typename TOut, bool SW, int TK>
static int launch_mfma_tile_t(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                              int ldx, int ldo, int out_cols, hipStream_t stream) {
    constexpr size_t lds = 2 * (size_t)(BM + BN) * (TK + 8) * sizeof(bf16_t);
    auto kernel = gemm_mfma_tile_kernel<BM, BN, WGM, WGN, TOut, SW, TK>;
    static hipError_t allowed = allow_lds(kernel, lds);
    if (allowed != hipSuccess) {
        tl_set_error("gemm_mfma_tile: cannot get %zu bytes of shared memory: %s", lds, hipGetErrorString(allowed));
        return TL_ERR_HIP;
    }
    dim3 grid(((M + BM - 1) / BM) * ((N + BN - 1) / BN)), block(64 * WGM * WGN);
    kernel<<<grid, block, lds, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (TOut*)out, M, N, K, ldx, ldo, out_cols);
    return TL_OK;
}

template <int BM, int BN, int WGM, int WGN, int TK = 32>
static int launch_mfma_tile(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                            int ldx, int ldo, int out_f32, hipStream_t stream) {
    if (out_f32) return launch_mfma_tile_t<BM, BN, WGM, WGN, float, false, TK>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream);
    return launch_mfma_tile_t<BM, BN, WGM, WGN, bf16_t, false, TK>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream);
}

// =====================================================================================
// The same product with the operands fetched straight into shared memory (K a multiple of 64).
//
// global_load_lds_dwordx4 moves 16 bytes per lane from memory into shared memory without passing
// through registers: one instruction of a wave fills 1 KB, eight rows of a 64-element slab.  A slab
// row is 128 bytes with no padding; piece c (16 bytes) of row r lies in slot c ^ ((r >> 1) & 7), so
// that the sixteen rows a quarter-wave reads for one MFMA operand fall on all 64 banks (measured:
// no bank conflicts).  The lane that fills slot s of row r therefore fetches piece s ^ ((r >> 1) & 7)
// of that row from memory.  STAGES slabs are in flight or in use: the slab STAGES - 1 ahead is
// requested into the buffer that a step has just finished with, and a step ends with a wait for
// this wave's requests of the next slab and one barrier.
// The requests are issued as assembly: the compiler orders every later shared-memory read behind
// a direct load it knows of (a full wait per slab), so the kernel keeps that order itself.  The
// address is a base that the wave shares and a 32-bit offset per lane.
__device__ __forceinline__ void load_to_lds_at(const void* base, unsigned offset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(offset), "s"(base), "s"(lds_addr) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_direct_loads() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

// Rows of one slab in shared memory: the BM rows of x and the BN rows of w, rounded up to what the waves'
// load instructions (64 lanes x 16 bytes each) fill between them.
constexpr int dl_slab_rows(int bm, int bn, int waves, int tk) {
    const int per = (64 / (tk / 8)) * waves;
    return (bm + bn + per - 1) / per * per;
}

template <int BM, int BN, int WGM, int WGN, int STAGES, typename TOut, bool SW = false, int TK = 64>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm_dl_tile_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                      const void* __restrict__ bias, int bias_f32,
                                                                      TOut* __restrict__ out, int M, int N, int K, int ldx, int ldo,
                                                                      int out_cols, int k_per_split) {
    static_assert(!SW || (BN / WGN) % 64 == 0, "the fused gate needs whole 64-row blocks per wave");
    static_assert(TK == 64 || TK == 32, "slabs of 64 or 32 columns");
    // A slab row holds PPR pieces of 16 bytes; one load instruction of a wave fills RPL rows.  With
    // slabs of 32 columns a row is 64 bytes and piece c of row r lies in slot c ^ ((r >> 2) & 3): the
    // sixteen rows a quarter-wave reads then fall on all 64 banks as well.  Half the slab is half the
    // shared memory per stage: twice as many stages fit, and a request has twice as long to arrive.
    constexpr int PPR = TK / 8, RPL = 64 / PPR;
#define DL_SWZ(r) (TK == 64 ? (((r) >> 1) & 7) : (((r) >> 2) & 3))
    // Split K (k_per_split > 0, a multiple of 64): blockIdx.y owns the columns [y * k_per_split, ...) of
    // x and w and writes its own [M, ldo] slab of partial sums to out; whoever reads them adds the slabs up.
    const int ldw = K;
    if (k_per_split > 0) {
        const int kb = blockIdx.y * k_per_split;
        x += kb;
        w += kb;
        out += (size_t)blockIdx.y * M * ldo;
        K = min(K - kb, k_per_split);
    }
    constexpr int NW = WGM * WGN;
    constexpr int WM = BM / WGM, WN = BN / WGN;          // wave tile
    constexpr int FM = WM / 32, FN = WN / 32;            // 32x32 blocks per wave
    constexpr int ROWS = BM + BN;
    constexpr int LROWS = dl_slab_rows(BM, BN, NW, TK);  // a slab's rows in shared memory: ROWS, rounded up so that ...
    constexpr int LOADS = LROWS / RPL / NW;              // ... every wave issues as many load instructions per slab (RPL rows each)
    static_assert(LOADS * (STAGES - 1) < 64, "outstanding loads must fit the counter");
    extern __shared__ __attribute__((aligned(16))) bf16_t lds_raw[];   // [STAGES][LROWS][TK]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    // tile order as in gemm_mfma_tile_kernel: each XCD walks 8 x 8 blocks of tiles out of its own L2
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int lid;
    {
        const int total = gridDim.x, xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
        lid = xcd * (total / 8) + min(xcd, total % 8) + idx;
    }
    int tm, tn;
    {
        const int per_group = 8 * tiles_n;
        const int first_m = (lid / per_group) * 8;
        const int rows = min(tiles_m - first_m, 8);
        tm = first_m + (lid % per_group) % rows;
        tn = (lid % per_group) / rows;
    }
    const int m0 = tm * BM, n0 = tn * BN;

    // Instruction j of this wave fills rows RPL (wave + j NW) .. + RPL of the stacked [x rows; w rows] slab.  Its
    // eight rows are all of x or all of w (BM is a multiple of RPL), so its address is a base the wave shares (the
    // tile's first row of x or of w, moved along K from step to step by scalar instructions) and a 32-bit offset per
    // lane that never changes: half the address registers of a 64-bit address per lane, and no vector addition per
    // request (2048 x 37888 x 3584: 500 -> 478 us).
    static_assert(BM % RPL == 0, "the rows of one request lie in one operand");
    int ldst[LOADS];
    unsigned soff[LOADS];
    unsigned of_x = 0;                                      // bit j: request j fetches rows of x
#pragma unroll
    for (int j = 0; j < LOADS; ++j) {
        const int base_row = RPL * (wave + j * NW);
        const int row = min(base_row + lane / PPR, ROWS - 1);      // (rows of the rounding: copies of the last row, never read)
        const int c = (lane % PPR) ^ DL_SWZ(row);
        if (row < BM) soff[j] = (unsigned)((min(m0 + row, M - 1) - m0) * ldx + c * 8) * 2;
        else soff[j] = (unsigned)((min(n0 + row - BM, N - 1) - n0) * ldw + c * 8) * 2;
        ldst[j] = __builtin_amdgcn_readfirstlane(base_row * TK * 2);
        of_x |= (unsigned)(base_row < BM) << j;
    }
    of_x = __builtin_amdgcn_readfirstlane(of_x);
    const bf16_t* xt = x + (size_t)m0 * ldx;
    const bf16_t* wt = w + (size_t)n0 * ldw;
    const unsigned lds_base = (unsigned)(uintptr_t)((void __attribute__((address_space(3)))*)lds_raw);

    f32x16_t acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int slabs = K / TK;
    const int fr = lane & 31, fh = lane >> 5;
    int arow[FM], brow[FN], akey[FM], bkey[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i) { arow[i] = wm * WM + i * 32 + fr; akey[i] = DL_SWZ(arow[i]); }
#pragma unroll
    for (int j = 0; j < FN; ++j) { brow[j] = BM + wn * WN + j * 32 + fr; bkey[j] = DL_SWZ(brow[j]); }
#undef DL_SWZ

    // The loop is a hand-laid pipeline; scheduling fences keep the compiler from undoing it.  A step
    // of TK columns has TK / 16 phases of FM * FN products.  A phase's memory instructions go between
    // its products, one product first: the operand reads of the next phase into the other register set,
    // so a read has a whole phase to arrive, and the wait before a phase's first product is for operands
    // asked for a phase ago with nothing younger outstanding.  (All reads first and then all products,
    // the wait at the loop's head came out as one for every read, the ones just issued too, and the 7B's fused
    // gate/up product at 2048 rows took 537 us instead of 487.)  The last phase of a step first waits for the
    // next slab and meets the other waves at the barrier (they have all read their last operands of this
    // slab by then); between its products go the first half of the requests for the slab STAGES - 1 ahead, into
    // the buffer just given up, and then the reads of the first operands of the next slab.  The other half of
    // the requests goes into the first phase of the next step: a compute unit's 64 requests in one phase hold
    // its waves up, whatever they fetch (requests of 4 bytes a lane cost the same; without any the loop ran a
    // sixth faster), and in two phases less so (2048 x 3584 x 18944: 392 -> 353 us; spread over three phases the
    // last ones arrive too late).  Past the end the last slab is requested again (nobody reads it), so the count
    // of requests in flight is the same in every step, which the wait relies on.
    Frag16 af[2][FM], bfr[2][FN];
    // requests of a slab issued in the last phase of a step; the rest in the next step's first.  (Not for the smallest tile,
    // four requests a wave and slab: split in two they made the decode step's products over K a fiftieth slower.)
    constexpr int L_LAST = LOADS >= 6 ? (LOADS + 1) / 2 : LOADS;
    auto request = [&](int slab, int j) {
        // (which operand request j fetches is known at compile time where the waves' requests cover whole multiples of x's rows)
        const bool from_x = BM % (RPL * NW) == 0 ? j < BM / (RPL * NW) : (bool)((of_x >> j) & 1);
        const bf16_t* from = (from_x ? xt : wt) + min(slab, slabs - 1) * TK;
        load_to_lds_at(from, soff[j], lds_base + (slab % STAGES) * LROWS * TK * 2 + ldst[j]);
    };
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st)
#pragma unroll
        for (int j = 0; j < LOADS; ++j) request(st, j);
    wait_direct_loads<(STAGES - 2) * LOADS>();
    __syncthreads();
#pragma unroll
    for (int j = 0; j < L_LAST; ++j) request(STAGES - 1, j);
#pragma unroll
    for (int i = 0; i < FM; ++i) af[0][i].u = *(const uint4*)(lds_raw + arow[i] * TK + ((fh ^ akey[i]) * 8));
#pragma unroll
    for (int j = 0; j < FN; ++j) bfr[0][j].u = *(const uint4*)(lds_raw + brow[j] * TK + ((fh ^ bkey[j]) * 8));
    __builtin_amdgcn_sched_barrier(0);

    constexpr int PHASES = TK / 16;
    constexpr int NM = FM * FN, NR = FM + FN;               // products and operand reads of a phase
    for (int sl = 0; sl < slabs; ++sl) {
        const bf16_t* cb = lds_raw + (sl % STAGES) * LROWS * TK;
#pragma unroll
        for (int kk = 0; kk < PHASES; ++kk) {
            const int cur = kk & 1, nxt = cur ^ 1;
            const bool last = kk + 1 == PHASES;
            const bf16_t* nb = last ? lds_raw + ((sl + 1) % STAGES) * LROWS * TK : cb;      // where the next phase's operands lie
            const int c = (last ? 0 : 2 * (kk + 1)) + fh;
            // this phase's requests [lfirst, lend) and the slab they fetch: in the last phase the slab that gets the
            // buffer given up now, in the first the rest of the slab that got the buffer given up a step ago
            const int lfirst = last ? 0 : L_LAST, lend = last ? L_LAST : kk == 0 ? LOADS : L_LAST;
            const int slab_of = last ? sl + STAGES : sl - 1 + STAGES;
            const int nl = lend - lfirst;
            const int ops = nl + NR;                                                         // memory instructions of this phase ...
            const int per = (ops + NM - 1) / NM;                                             // ... and how many follow each product
            if (last) {
                wait_direct_loads<(STAGES - 2) * LOADS>();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (NM == 1) {
                // One product a phase (the smallest tile): a phase's memory instructions first, then its product, which
                // covers them; but for the step's first phase, whose product comes first so that the wait at the loop's
                // head is for that product's operands alone.
                if (kk == 0) {
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][0].v, af[cur][0].v, acc[0][0], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int op = 0; op < ops; ++op) {
                    const int r = op - nl;
                    if (r < 0) request(slab_of, lfirst + op);
                    else if (r < FM) af[nxt][r].u = *(const uint4*)(nb + arow[r] * TK + ((c ^ akey[r]) * 8));
                    else bfr[nxt][r - FM].u = *(const uint4*)(nb + brow[r - FM] * TK + ((c ^ bkey[r - FM]) * 8));
                }
                __builtin_amdgcn_sched_barrier(0);
                if (kk > 0) {
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][0].v, af[cur][0].v, acc[0][0], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                }
                continue;
            }
            int op = 0;
#pragma unroll
            for (int q = 0; q < NM; ++q) {
                acc[q / FN][q % FN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[cur][q % FN].v, af[cur][q / FN].v, acc[q / FN][q % FN], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < per; ++e, ++op) {
                    if (op >= ops) break;
                    const int r = op - nl;
                    if (r < 0) request(slab_of, lfirst + op);
                    else if (r < FM) af[nxt][r].u = *(const uint4*)(nb + arow[r] * TK + ((c ^ akey[r]) * 8));
                    else bfr[nxt][r - FM].u = *(const uint4*)(nb + brow[r - FM] * TK + ((c ^ bkey[r - FM]) * 8));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    wait_direct_loads<0>();

    // The products are taken as weight block times x block, so of a 32x32 block a lane holds one
    // row of x, m = lane % 32, and sixteen output columns n = 8 (v / 4) + 4 (lane / 32) + v % 4:
    // four neighbours at a time.  With the fused gate, even blocks hold gate columns and the next
    // block the up columns of the same 32 outputs.
    const int lm = lane & 31, half = lane >> 5;
    constexpr int WNO = SW ? WN / 2 : WN;                   // output columns of a wave tile
    constexpr int FNO = SW ? FN / 2 : FN;                   // and its blocks of 32 of them
    const int cols = SW ? out_cols : N;                     // output columns in all
    const int c0 = (SW ? n0 / 2 : n0) + wn * WNO;           // first output column and row of this wave
    const int r0 = m0 + wm * WM;
    auto value = [&](int i, int jo, int v) -> float {
        if constexpr (SW) return silu_mul(acc[i][2 * jo][v], acc[i][2 * jo + 1][v]);
        else return acc[i][jo][v];
    };
    auto bias_at = [&](int n) -> float { return (!SW && bias && n < cols) ? load_vec(bias, bias_f32, n) : 0.f; };

    if constexpr (sizeof(TOut) == 2) {
        if (cols % 8 == 0 && ldo % 8 == 0 && ((uintptr_t)out % 16) == 0) {
            // bfloat16 rows that can be stored in 16-byte pieces: the wave lays its tile out row by
            // row in shared memory (the slab buffers are free now; 16-byte piece c of row r in slot
            // c ^ (r % CX) against bank conflicts) and stores it in whole rows, 64 lanes times 16
            // bytes per instruction, instead of two bytes per lane and store.
            constexpr int C = WNO / 8;
            constexpr int CX = C & -C;                       // the slots are exchanged within groups of CX, a power of two
            static_assert((WM * C) % 64 == 0, "the rows of a wave tile must divide over its lanes");
            static_assert(BM * (SW ? BN / 2 : BN) <= STAGES * ROWS * TK, "the result tile must fit the slab buffers");
            __syncthreads();
            bf16_t* stage = lds_raw + wave * (WM * WNO);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int jo = 0; jo < FNO; ++jo)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int n = jo * 32 + 8 * g + 4 * half;
                        bf16_t h[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) h[e] = from_float<bf16_t>(value(i, jo, 4 * g + e) + bias_at(c0 + n + e));
                        uint2 packed;
                        packed.x = (uint32_t)h[0].bits | ((uint32_t)h[1].bits << 16);
                        packed.y = (uint32_t)h[2].bits | ((uint32_t)h[3].bits << 16);
                        const int row = i * 32 + lm;
                        *(uint2*)(stage + row * WNO + (((n >> 3) ^ (row & (CX - 1))) * 8) + (n & 4)) = packed;
                    }
            // (one wave's shared-memory accesses are carried out in order: no wait in between)
#pragma unroll
            for (int q = 0; q < WM * C / 64; ++q) {
                const int idx = q * 64 + lane;
                const int row = idx / C, piece = idx % C;
                const uint4 val = *(const uint4*)(stage + row * WNO + ((piece ^ (row & (CX - 1))) * 8));
                const int m = r0 + row, n = c0 + piece * 8;
                if (m < M && n < cols) *(uint4*)((bf16_t*)out + (size_t)m * ldo + n) = val;
            }
            return;
        }
    }
    const bool quads = sizeof(TOut) == 4 && cols % 4 == 0 && ldo % 4 == 0 && ((uintptr_t)out % 16) == 0;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
        const int m = r0 + i * 32 + lm;
        if (m >= M) continue;
#pragma unroll
        for (int jo = 0; jo < FNO; ++jo)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = c0 + jo * 32 + 8 * g + 4 * half;
                if (quads) {
                    if (n < cols) {
                        float4 f;
                        f.x = value(i, jo, 4 * g) + bias_at(n);
                        f.y = value(i, jo, 4 * g + 1) + bias_at(n + 1);
                        f.z = value(i, jo, 4 * g + 2) + bias_at(n + 2);
                        f.w = value(i, jo, 4 * g + 3) + bias_at(n + 3);
                        *(float4*)((float*)out + (size_t)m * ldo + n) = f;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < cols) out[(size_t)m * ldo + n + e] = from_float<TOut>(value(i, jo, 4 * g + e) + bias_at(n + e));
                }
            }
    }
}

// Tile shapes of the direct-load kernel and which one a product gets.  Estimate per shape: the
// tiles are dealt to 256 compute units, each works through ceil(tiles / 256) of them one after
// the other; a tile takes a fixed time (filling the pipeline, storing the result) plus its
// products at the rate one compute unit reaches with that shape (fitted to measurements at
// 2048 rows against the Qwen2.5-7B and 14B matrices, K from 3584 to 18944).
// (DL_128x128_S4: 128 x 128 with four slabs in shared memory, one work-group to a compute unit: for products of up
// to 128 rows split over K, where what counts is how many bytes of weights a work-group has on their way; measured
// at 128 rows against the best other tile: 3584 x 18944 48.8 -> 37.1 us, 3584 x 3584 18.6 -> 15.8, 5120 x 5120 29.7 -> 21.4)
// (DL_256x320: eight waves of 64 x 160, 246 registers, 144 KB of slabs; float slabs of a split K only, since a bfloat16
// result tile of 160 KB does not fit its slab buffers.  It is there for thousands of rows against a matrix 5120 wide:
// 2048 rows are 160 tiles of 256 x 256, which leave 96 of 256 compute units idle, and 128 of these, which with K in
// two halves are one round of 256 work-groups.  Measured at 2048 rows, slabs written: 5120 x 27648 504 us against
// 651 whole and 573 in three parts of 256 x 256; 5120 x 13824 263 against 324 and 306; 5120 x 5120 112 against 140
// and 132.  Its rate here is the one it reaches with all compute units busy, lower than a tile's that runs on 160.)
// (DL_256x160: four waves of 64 x 160, for matrices 5120 wide as well: 2048 rows are 256 tiles, one to a compute
// unit, and 4096 rows two rounds of them where tiles of 256 x 256 take one and a quarter.  A compute unit gets through
// a slab of it hardly faster than through one of 256 x 256 (what a slab costs is mostly its requests, 52 against 64,
// not its products, 40 against 64), so it wins only where it fills rounds that the square tile leaves part empty.
// Measured, whole products: 2048 x 5120 x 13824 261 us against 274-296; 2048 x 5120 x 5120 97 against 106; at 4096
// rows 499 against 585 and 202 against 239; 4096 x 4608 x 3584 130 against 158.  Eight waves of 32 x 160: 265, 99.)
enum DlTile { DL_64x64, DL_64x256, DL_128x128, DL_128x256, DL_256x128, DL_192x256, DL_256x192, DL_256x256, DL_64x128, DL_128x128_S4, DL_64x192, DL_128x192, DL_64x320, DL_256x320, DL_256x160, DL_TILES };
static const int DL_BM[DL_TILES] = {64, 64, 128, 128, 256, 192, 256, 256, 64, 128, 64, 128, 64, 256, 256};
static const int DL_BN[DL_TILES] = {64, 256, 128, 256, 128, 256, 192, 256, 128, 128, 192, 192, 320, 320, 160};
static const double DL_RATE[DL_TILES] = {2.45e12, 3.3e12, 4.2e12, 4.6e12, 4.8e12, 5.2e12, 5.2e12, 6.1e12, 2.1e12, 4.2e12, 3.0e12, 4.4e12, 3.5e12, 5.5e12, 4.3e12};   // FLOP/s of one compute unit
static const double DL_FIXED[DL_TILES] = {2.7e-6, 11.5e-6, 5.5e-6, 11e-6, 15e-6, 6e-6, 8e-6, 14e-6, 5e-6, 4.5e-6, 9e-6, 9e-6, 12e-6, 10e-6, 10e-6};       // seconds per tile

// Seconds for `groups` work-groups of tile t over k columns each.  The two smallest tiles run two
// to a compute unit: each then works at half the unit's rate, and one that has a unit to itself
// (not more work-groups than units) at about 0.62 of it.  With few rows the products wait for the
// operands: a compute unit fills its shared memory at about 40 GB/s, and a work-group draws its BN
// rows of weights and its BM rows of x alike (x as often as there are tiles along N: with 64 x 64 tiles
// as many bytes of x as of weights).  Measured at 17-64 rows: on the 14B's gate/up matrix 108 work-groups
// of 64 x 256 take 81 us, 216 of 64 x 128 take 56-59, 432 of 64 x 64 (two to a unit) 59-68; on the 7B's
// 148 of 64 x 256 take 55-60 and 592 of 64 x 64 take 57-66; on the LM head at 128 rows 594 of 128 x 256
// take 239 and 1188 of 128 x 128 take 266.  `weights_only`: the estimates of plan_dl_split (whether and how to
// split K over work-groups, a few hundred rows against a narrow matrix) count the weights alone, at 32 GB/s,
// which is what its plans were fitted with: with x counted they came out a tenth slower at 512 rows against
// the down projections (87 against 82 us on the 7B's).
static double dl_estimate(DlTile t, long groups, int k, bool weights_only = false) {
    const bool pairs = t == DL_64x64 || t == DL_128x128;
    const double products = 2.0 * DL_BM[t] * DL_BN[t] * k;
    const double stream = weights_only ? 2.0 * DL_BN[t] * k / 32e9 : 2.0 * (DL_BN[t] + DL_BM[t]) * k / 40e9;
    const int cus = TL_COMPUTE_UNITS;
    if (!pairs) return (double)((groups + cus - 1) / cus) * fmax(products / DL_RATE[t] + DL_FIXED[t], stream);
    const double rate = groups > cus ? DL_RATE[t] / 2 : DL_RATE[t] * 0.62;
    // (a single round of 128 x 128 tiles runs a tenth behind this estimate: measured on the fused gate/up
    // products of the 7B, 14B and 32B at 96 to 512 rows, where it otherwise displaced 128 x 256 tiles
    // that were up to a fifth faster)
    const double lag = (t == DL_128x128 && groups <= 2 * cus) ? 1.1 : 1.0;
    return lag * (double)((groups + 2 * cus - 1) / (2 * cus)) * fmax(products / rate + DL_FIXED[t], groups > cus ? 2 * stream : stream);
}

static DlTile pick_dl_tile(int M, int N, int K, bool sw, double* estimate = nullptr, bool weights_only = false) {
    DlTile best = DL_128x128;
    double best_t = 1e30;
    for (int t = 0; t < DL_TILES; ++t) {
        if (sw && (t == DL_64x64 || t == DL_256x192 || t == DL_64x320 || t == DL_256x160)) continue;      // a wave of the fused gate needs whole 64-row blocks of weights
        if (t == DL_256x320) continue;      // float slabs of partial sums only: a bfloat16 result tile of 160 KB does not fit its slab buffers
        const long tiles = (long)((M + DL_BM[t] - 1) / DL_BM[t]) * ((N + DL_BN[t] - 1) / DL_BN[t]);
        if (t == DL_128x128_S4 && (tiles > TL_COMPUTE_UNITS || M > 128)) continue;      // one round of work-groups, every weight drawn once
        // (the split planner's unsplit baseline is fitted without the 192-wide tiles: with them it kept 512 rows against the
        // 14B's query/key/value matrix whole, 74.8 us, where it used to split K, 53.9 us)
        if (weights_only && (t == DL_64x192 || t == DL_128x192 || t == DL_64x320)) continue;
        const double est = dl_estimate((DlTile)t, tiles, K, weights_only);
        if (est < best_t) { best_t = est; best = (DlTile)t; }
    }
    if (estimate) *estimate = best_t;
    return best;
}

// More than 64 rows against a matrix whose output tiles leave compute units idle (a few hundred rows
// of a prompt portion against the down projection, say): K split over `parts` work-groups per tile
// into float slabs that the consumer adds up.  Only the tiles that have a compute unit to themselves
// are considered; the slabs cost their bytes once written and once read.  parts == 1: no split pays.
struct DlSplit { DlTile tile; int parts; int k_per; };
static DlSplit plan_dl_split(int M, int N, int K) {
    double best_t;
    DlSplit best{pick_dl_tile(M, N, K, false, &best_t, true), 1, 0};
    best_t += (double)M * N * 2 * 2 / 3e12;
    const int steps = K / 64;
    static const DlTile alone[] = {DL_128x128_S4, DL_128x256, DL_256x128, DL_192x256, DL_256x192, DL_256x256, DL_256x320, DL_64x64};
    for (DlTile t : alone) {
        const long tiles = (long)((M + DL_BM[t] - 1) / DL_BM[t]) * ((N + DL_BN[t] - 1) / DL_BN[t]);
        for (int P = 2; P <= 8 && K / P >= 512; ++P) {
            const int k_per = ((steps + P - 1) / P) * 64;
            if ((K + k_per - 1) / k_per != P) continue;
            if (t == DL_128x128_S4 && tiles * P > TL_COMPUTE_UNITS) continue;       // measured in one round of work-groups only
            // (the small tile as for up to 64 rows, one work-group to a compute unit: 128 rows against the 7B's output
            // projection 13.0 us in two parts where four parts of 128 x 128 take 17.0)
            if (t == DL_64x64 && (M > 128 || tiles * P > TL_COMPUTE_UNITS)) continue;
            // (a tenth on top: float slabs leave the kernel more slowly than the estimate's bfloat16 rows)
            const double est = 1.1 * dl_estimate(t, tiles * P, k_per, true) + (double)P * M * N * 4 * 2 / 3e12;
            if (est < best_t) { best_t = est; best = DlSplit{t, P, k_per}; }
        }
    }
    return best;
}

// parts > 1 (float results only): K is split into `parts` ranges of k_per columns and out holds that many [M, ldo] slabs.
template <int BM, int BN, int WGM, int WGN, int STAGES, typename TOut, bool SW, int TK = 64>
static int launch_dl_tile_t(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                            int ldx, int ldo, int out_cols, hipStream_t stream, int parts = 1, int k_per = 0) {
    constexpr size_t lds = (size_t)STAGES * dl_slab_rows(BM, BN, WGM * WGN, TK) * TK * sizeof(bf16_t);
    // (a lane's offset from its tile's first row is kept in 32 bits)
    TL_REQUIRE((long)(BM > BN ? BM : BN) * (ldx > K ? ldx : K) * 2 < (1L << 31), "gemm_dl_tile: rows of %d elements are too long", ldx > K ? ldx : K);
    auto kernel = gemm_dl_tile_kernel<BM, BN, WGM, WGN, STAGES, TOut, SW, TK>;
    static hipError_t allowed = allow_lds(kernel, lds);
    if (allowed != hipSuccess) {
        tl_set_error("gemm_dl_tile: cannot get %zu bytes of shared memory: %s", lds, hipGetErrorString(allowed));
        return TL_ERR_HIP;
    }
    dim3 grid(((M + BM - 1) / BM) * ((N + BN - 1) / BN), parts), block(64 * WGM * WGN);
    kernel<<<grid, block, lds, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (TOut*)out, M, N, K, ldx, ldo, out_cols,
                                         parts > 1 ? k_per : 0);
    return TL_OK;
}

template <typename TOut, bool SW>
static int launch_dl_tile(DlTile tile, const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                          int ldx, int ldo, int out_cols, hipStream_t stream, int parts = 1, int k_per = 0) {
    switch (tile) {
    case DL_64x64:
        if constexpr (!SW) return launch_dl_tile_t<64, 64, 2, 2, 4, TOut, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
        else break;
    case DL_64x256: return launch_dl_tile_t<64, 256, 1, 4, 3, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_128x128: return launch_dl_tile_t<128, 128, 2, 2, 2, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_128x128_S4: return launch_dl_tile_t<128, 128, 2, 2, 4, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_128x256: return launch_dl_tile_t<128, 256, 2, 4, 3, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_256x128: return launch_dl_tile_t<256, 128, 4, 2, 3, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_64x128: return launch_dl_tile_t<64, 128, 1, 2, 3, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_64x192: return launch_dl_tile_t<64, 192, 1, 3, 4, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_64x320:
        if constexpr (!SW) return launch_dl_tile_t<64, 320, 1, 5, 3, TOut, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
        else break;
    case DL_128x192: return launch_dl_tile_t<128, 192, 2, 3, 3, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_192x256: return launch_dl_tile_t<192, 256, 2, 4, 2, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_256x192:
        if constexpr (!SW) return launch_dl_tile_t<256, 192, 4, 2, 2, TOut, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
        else break;
    case DL_256x256: return launch_dl_tile_t<256, 256, 4, 2, 2, TOut, SW>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
    case DL_256x160:
        if constexpr (!SW) return launch_dl_tile_t<256, 160, 4, 1, 2, TOut, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
        else break;
    case DL_256x320:
        if constexpr (!SW && sizeof(TOut) == 4) return launch_dl_tile_t<256, 320, 4, 2, 2, float, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_cols, stream, parts, k_per);
        else break;
    default: break;
    }
    tl_set_error("gemm_dl_tile: no instance of tile %d", (int)tile);
    return TL_ERR_ARG;
}

// One named tile shape of the many-rows kernel (tests cover each; tuning times them).
extern "C" int tl_gemm_tile_variant(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                                    int M, int N, int K, int ldx, int ldo, int out_f32, int BM, int BN, int TK, hipStream_t stream) {
    TL_REQUIRE(M > 0 && K % 8 == 0 && ldx % 8 == 0, "gemm_tile: needs M > 0 and K, ldx multiples of 8");
    int rc = -1;
#define TL_TILE_CASE(bm, bn, gm, gn, tk) \
    if (BM == bm && BN == bn && TK == tk) rc = launch_mfma_tile<bm, bn, gm, gn, tk>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
    // the tile shapes pick_tile can choose
    TL_TILE_CASE(128, 128, 2, 2, 32) TL_TILE_CASE(128, 128, 2, 2, 64)
    TL_TILE_CASE(64, 128, 2, 2, 64) TL_TILE_CASE(256, 256, 4, 2, 64)
#undef TL_TILE_CASE
    TL_REQUIRE(rc != -1, "gemm_tile: no instance BM=%d BN=%d TK=%d", BM, BN, TK);
    if (rc != TL_OK) return rc;
    TL_CHECK_LAUNCH("gemm_mfma_tile");
    return TL_OK;
}

// One named tile shape of the direct-load kernel (tests cover each; tuning times them).
extern "C" int tl_gemm_direct_variant(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                                      int M, int N, int K, int ldx, int ldo, int out_f32, int BM, int BN, hipStream_t stream) {
    TL_REQUIRE(M > 0 && K % 64 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
               "gemm_direct: needs M > 0, K a multiple of 64 and 16-byte aligned rows");
    int tile = -1;
    for (int t = 0; t < DL_TILES; ++t)
        if (DL_BM[t] == BM && DL_BN[t] == BN && t != DL_128x128_S4) tile = t;
    TL_REQUIRE(tile >= 0, "gemm_direct: no tile of %d x %d", BM, BN);
    const int rc = out_f32 ? launch_dl_tile<float, false>((DlTile)tile, x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream)
                           : launch_dl_tile<bf16_t, false>((DlTile)tile, x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream);
    if (rc != TL_OK) return rc;
    TL_CHECK_LAUNCH("gemm_dl_tile");
    return TL_OK;
}

// The fused gate/up product (see tl_gemm_swiglu) on one named tile shape; for tests and tuning.
extern "C" int tl_gemm_swiglu_direct_variant(const void* x, const void* w, void* out, int M, int I, int K, int ldx, int ldo,
                                             int BM, int BN, hipStream_t stream) {
    TL_REQUIRE(M > 0 && I > 0 && K % 64 == 0 && ldx % 8 == 0 && ldo >= I && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
               "gemm_swiglu_direct: needs M > 0, K a multiple of 64 and 16-byte aligned rows");
    int tile = -1;
    for (int t = 0; t < DL_TILES; ++t)
        if (DL_BM[t] == BM && DL_BN[t] == BN && t != DL_128x128_S4 && t != DL_64x64 && t != DL_256x192 && t != DL_64x320 && t != DL_256x320 && t != DL_256x160) tile = t;
    TL_REQUIRE(tile >= 0, "gemm_swiglu_direct: no tile of %d x %d with the fused gate", BM, BN);
    const int N = ((I + 31) / 32) * 64;
    const int rc = launch_dl_tile<bf16_t, true>((DlTile)tile, x, w, nullptr, 0, out, M, N, K, ldx, ldo, I, stream);
    if (rc != TL_OK) return rc;
    TL_CHECK_LAUNCH("gemm_dl_tile");
    return TL_OK;
}

// One tile shape with K split into `parts` (float slabs [parts, M, N]); for tests and tuning.
// stages == 4 with 128 x 128: the four-slab instance.
extern "C" int tl_gemm_direct_split_variant(const void* x, const void* w, void* out, int M, int N, int K, int ldx,
                                            int BM, int BN, int parts, int stages, hipStream_t stream) {
    TL_REQUIRE(M > 0 && K % 64 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0 && parts >= 1,
               "gemm_direct_split: needs M > 0, K a multiple of 64 and 16-byte aligned rows");
    int tile = -1;
    for (int t = 0; t < DL_TILES; ++t)
        if (DL_BM[t] == BM && DL_BN[t] == BN && (t == DL_128x128_S4) == (stages == 4)) tile = t;
    TL_REQUIRE(tile >= 0, "gemm_direct_split: no tile of %d x %d with %d stages", BM, BN, stages);
    const int steps = K / 64;
    const int k_per = ((steps + parts - 1) / parts) * 64;
    TL_REQUIRE((K + k_per - 1) / k_per == parts, "gemm_direct_split: %d parts leave one empty (K=%d)", parts, K);
    const int rc = launch_dl_tile<float, false>((DlTile)tile, x, w, nullptr, 0, out, M, N, K, ldx, N, 0, stream, parts, k_per);
    if (rc != TL_OK) return rc;
    TL_CHECK_LAUNCH("gemm_direct_split");
    return TL_OK;
}

static bool skinny_fits(const void* x, const void* w, int M, int K, int ldx) {
    return M <= 64 && K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
}

// out = x w^T (+ bias) in the engine's dtype: picks the kernel for the shape.
//   bfloat16, aligned, M <= 64  -> gemm_skinny (matrix cores, weight streaming), except that
//                                  33..64 rows against a wide matrix go to the tile kernel
//   bfloat16, aligned, K a multiple of 64, M > 32 (M > 8 against a wide matrix) -> gemm_dl_tile
//                                  (matrix cores, operands straight into shared memory)
//   bfloat16, aligned, M > 64   -> gemm_mfma_tile (matrix cores, shared-memory tiles)
//   32-bit, aligned, M <= 16    -> gemv_f32 (true 32-bit arithmetic, weight streaming)
//   32-bit, aligned, M > 16     -> gemm_f32_mfma (true 32-bit arithmetic on the matrix cores)
//   everything else             -> gemm_tile (true 32-bit arithmetic)
extern "C" int tl_gemm(const void* x, const void* w, const void* bias, int bias_f32, void* out,
                       int M, int N, int K, int ldx, int ldo, int dtype, int out_f32, hipStream_t stream) {
    TL_REQUIRE(M >= 0 && N > 0 && K > 0 && ldx >= K && ldo >= N, "gemm: bad sizes M=%d N=%d K=%d ldx=%d ldo=%d", M, N, K, ldx, ldo);
    if (M == 0) return TL_OK;
    const bool aligned = K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0;
    // (measured at 17-32 rows: against a wide matrix the tile kernel is far ahead, 60 against 85-107 us
    // on gate/up and 200 against 310-400 us on the LM head; against a narrow one the skinny kernel wins)
    if (dtype == TL_DT_BF16 && aligned && K % 64 == 0 && (M > 32 || (M > 8 && N >= 16384))) {
        int rc = out_f32 ? launch_dl_tile<float, false>(pick_dl_tile(M, N, K, false), x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream)
                         : launch_dl_tile<bf16_t, false>(pick_dl_tile(M, N, K, false), x, w, bias, bias_f32, out, M, N, K, ldx, ldo, 0, stream);
        if (rc != TL_OK) return rc;
        TL_CHECK_LAUNCH("gemm_dl_tile");
        return TL_OK;
    }
    if (dtype == TL_DT_BF16 && aligned && (M > 64 || (M > 32 && N >= 16384))) {
        int rc;
        switch (pick_tile(M, N)) {
        case TILE_256x256: rc = launch_mfma_tile<256, 256, 4, 2, 64>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream); break;
        case TILE_128x128_K32: rc = launch_mfma_tile<128, 128, 2, 2, 32>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream); break;
        case TILE_128x128_K64: rc = launch_mfma_tile<128, 128, 2, 2, 64>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream); break;
        default: rc = launch_mfma_tile<64, 128, 2, 2, 64>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream); break;
        }
        if (rc != TL_OK) return rc;
        TL_CHECK_LAUNCH("gemm_mfma_tile");
        return TL_OK;
    }
    if (dtype == TL_DT_BF16 && skinny_fits(x, w, M, K, ldx)) {
        if (M <= 16) pick_skinny<1>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
        else if (M <= 32) pick_skinny<2>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
        else pick_skinny<4>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, out_f32, stream);
        TL_CHECK_LAUNCH("gemm_skinny");
        return TL_OK;
    }
    if (dtype == TL_DT_F32 && gemv_f32_fits(x, w, M, K, ldx)) {
        launch_gemv_f32(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
        TL_CHECK_LAUNCH("gemv_f32");
        return TL_OK;
    }
    if (dtype == TL_DT_F32 && gemm_f32_mfma_fits(x, w, M, K, ldx)) {
        launch_gemm_f32_mfma(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, stream);
        TL_CHECK_LAUNCH("gemm_f32_mfma");
        return TL_OK;
    }
    return tl_gemm_general(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, dtype, out_f32, stream);
}

// The fused query/key/value projection of up to 16 rows: out[:, :q_heads * head_dim] = rotated queries,
// rotated keys and values go to their pages (see RopeArgs; the weight rows of every query and key head
// are in the pair layout).  Returns TL_NOT_FUSED (nothing launched) for shapes it is not built for;
// the caller then runs the product and the rotation as two kernels.
#define TL_NOT_FUSED 100
template <int KS, bool XL, int R = 1>
static void launch_skinny_rope(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                               int ldx, int ldo, const RopeArgs& ra, hipStream_t stream, int rows_per_strip = 0) {
    const int rps = rows_per_strip > 0 ? rows_per_strip : 16 * R;
    dim3 grid((N + rps - 1) / rps), block(KS * 64);
    const size_t lds = (size_t)KS * R * 1024 + (XL ? (size_t)M * (K + 8) * 2 : 0);
    auto kernel = gemm_skinny_kernel<R, 1, KS, bf16_t, false, XL, 2, true>;
    if (XL) { static hipError_t allowed = allow_lds(kernel, 96 * 1024); (void)allowed; }
    kernel<<<grid, block, lds, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, bias_f32, (bf16_t*)out, M, N, K, ldx, ldo, 0, 0, rps, 0, ra, NormArgs{});
}

extern "C" int tl_gemm_partials_pay(int M, int N, int K);

extern "C" int tl_gemm_rope(const void* x, const void* w, const void* bias, int bias_f32, void* out, int M, int N, int K,
                            int ldx, int ldo, const void* positions, const void* inv_freq, const void* token_req,
                            const void* block_table, int bt_stride, void* k_plane, void* v_plane, int page,
                            int q_heads, int kv_heads, int head_dim, hipStream_t stream) {
    TL_REQUIRE(M > 0 && N > 0 && K > 0 && ldx >= K && ldo >= q_heads * head_dim, "gemm_rope: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_REQUIRE(positions && inv_freq && head_dim % 4 == 0 && q_heads >= 0 && kv_heads >= 0, "gemm_rope: needs positions, frequencies and a head size that is a multiple of 4");
    TL_REQUIRE((k_plane == nullptr) == (v_plane == nullptr) && (!k_plane || (token_req && block_table && page > 0 && bt_stride > 0)),
               "gemm_rope: the cache write needs both planes, the block table and the requests of the rows");
    TL_REQUIRE(N == (q_heads + (k_plane ? 2 * kv_heads : 0)) * head_dim, "gemm_rope: %d output columns do not match the heads", N);
    const int strips = (N + 15) / 16, ks = strips >= 1024 ? 16 : 8;
    // (from 9 rows on the product split over K on the tile kernel plus the rotation kernel that adds its slabs up
    // is ahead where that split is to be had: 4608 x 3584 at 16 rows 14.5 against 17.0 us, at 8 rows 14.8 against 14.0)
    if (M > 16 || (M > 8 && tl_gemm_partials_pay(M, N, K)) || !skinny_fits(x, w, M, K, ldx) || N % 16 || ldo % 4 || ((uintptr_t)out % 8) || K / 64 / ks >= 16 ||
        (k_plane && (((uintptr_t)k_plane % 8) || head_dim % 4)))
        return TL_NOT_FUSED;
    RopeArgs ra;
    ra.positions = (const int*)positions; ra.inv_freq = (const float*)inv_freq; ra.token_req = (const int*)token_req;
    ra.block_table = (const int*)block_table; ra.k_plane = (bf16_t*)k_plane; ra.v_plane = (bf16_t*)v_plane;
    ra.bt_stride = bt_stride; ra.page = page > 0 ? page : 1; ra.q_heads = q_heads; ra.kv_heads = k_plane ? kv_heads : 0; ra.head_dim = head_dim;
    const bool xl = M > 1 && (size_t)M * (K + 8) * 2 <= SKINNY_XL_MAX_BYTES;
    int blocks = 1;
    const int rows = ks == 8 ? balanced_rows(N, &blocks) : 0;
    if (rows > 0 && blocks == 2) { if (xl) launch_skinny_rope<8, true, 2>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, ra, stream, rows); else launch_skinny_rope<8, false, 2>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, ra, stream, rows); }
    else if (ks == 8) { if (xl) launch_skinny_rope<8, true>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, ra, stream, rows); else launch_skinny_rope<8, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, ra, stream, rows); }
    else { if (xl) launch_skinny_rope<16, true>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, ra, stream); else launch_skinny_rope<16, false>(x, w, bias, bias_f32, out, M, N, K, ldx, ldo, ra, stream); }
    TL_CHECK_LAUNCH("gemm_rope");
    return TL_OK;
}

// What a fused norm needs to be right: whole 16-byte pieces everywhere, two pieces per thread at most.
static bool norm_fits(const NormArgs& na, int K, int threads) {
    return K % 8 == 0 && K <= 16 * threads && na.residual && na.residual_out && na.residual != na.residual_out && na.weight &&
           ((uintptr_t)na.residual % 16) == 0 && ((uintptr_t)na.residual_out % 16) == 0 && ((uintptr_t)na.weight % 16) == 0 &&
           ((uintptr_t)na.pending % 16) == 0 && (na.parts == 0 || na.part_stride % 4 == 0) && na.parts >= 0 && na.parts <= 64;
}

static NormArgs norm_args(const void* residual, void* residual_out, const void* pending, int parts, long part_stride,
                          const void* weight, int weight_f32, float eps) {
    NormArgs na;
    na.residual = (const float*)residual; na.residual_out = (float*)residual_out; na.pending = pending;
    na.weight = weight; na.part_stride = (size_t)part_stride; na.parts = parts; na.weight_f32 = weight_f32; na.eps = eps;
    return na;
}

// tl_gemm_rope for one row whose x is the norm of the residual stream, made inside the kernel (see NormArgs):
// pending is bfloat16 [K] (parts == 0), float [parts][part_stride] or null.  Returns TL_NOT_FUSED (nothing
// launched) for shapes it is not built for; the caller then runs the norm and tl_gemm_rope.
extern "C" int tl_gemm_rope_normed(const void* residual, void* residual_out, const void* pending, int parts, long part_stride,
                                   const void* norm_weight, int norm_weight_f32, float eps,
                                   const void* w, const void* bias, int bias_f32, void* out, int N, int K, int ldo,
                                   const void* positions, const void* inv_freq, const void* token_req,
                                   const void* block_table, int bt_stride, void* k_plane, void* v_plane, int page,
                                   int q_heads, int kv_heads, int head_dim, hipStream_t stream) {
    TL_REQUIRE(N > 0 && K > 0 && ldo >= q_heads * head_dim, "gemm_rope_normed: bad sizes N=%d K=%d", N, K);
    TL_REQUIRE(positions && inv_freq && head_dim % 4 == 0 && q_heads >= 0 && kv_heads >= 0, "gemm_rope_normed: needs positions, frequencies and a head size that is a multiple of 4");
    TL_REQUIRE((k_plane == nullptr) == (v_plane == nullptr) && (!k_plane || (token_req && block_table && page > 0 && bt_stride > 0)),
               "gemm_rope_normed: the cache write needs both planes, the block table and the request of the row");
    TL_REQUIRE(N == (q_heads + (k_plane ? 2 * kv_heads : 0)) * head_dim, "gemm_rope_normed: %d output columns do not match the heads", N);
    const NormArgs na = norm_args(residual, residual_out, pending, parts, part_stride, norm_weight, norm_weight_f32, eps);
    const int strips = (N + 15) / 16, ks = strips >= 1024 ? 16 : 8;
    if (!norm_fits(na, K, ks * 64) || ((uintptr_t)w % 16) || N % 16 || ldo % 4 || ((uintptr_t)out % 8) || K / 64 / ks >= 16 ||
        (k_plane && (((uintptr_t)k_plane % 8) || head_dim % 4)))
        return TL_NOT_FUSED;
    RopeArgs ra;
    ra.positions = (const int*)positions; ra.inv_freq = (const float*)inv_freq; ra.token_req = (const int*)token_req;
    ra.block_table = (const int*)block_table; ra.k_plane = (bf16_t*)k_plane; ra.v_plane = (bf16_t*)v_plane;
    ra.bt_stride = bt_stride; ra.page = page > 0 ? page : 1; ra.q_heads = q_heads; ra.kv_heads = k_plane ? kv_heads : 0; ra.head_dim = head_dim;
    int blocks = 1;
    const int rows = ks == 8 ? balanced_rows(N, &blocks) : 0;
    dim3 grid(rows > 0 ? (N + rows - 1) / rows : strips);
    const size_t lds = (size_t)ks * blocks * 1024 + (size_t)(K + 8) * 2;
    if (rows > 0 && blocks == 2)
        gemm_skinny_kernel<2, 1, 8, bf16_t, false, true, 2, true, true><<<grid, dim3(8 * 64), lds, stream>>>(
            nullptr, (const bf16_t*)w, bias, bias_f32, (bf16_t*)out, 1, N, K, K, ldo, 0, 0, rows, 0, ra, na);
    else if (ks == 8)
        gemm_skinny_kernel<1, 1, 8, bf16_t, false, true, 2, true, true><<<grid, dim3(8 * 64), lds, stream>>>(
            nullptr, (const bf16_t*)w, bias, bias_f32, (bf16_t*)out, 1, N, K, K, ldo, 0, 0, rows, 0, ra, na);
    else
        gemm_skinny_kernel<1, 1, 16, bf16_t, false, true, 2, true, true><<<grid, dim3(16 * 64), lds, stream>>>(
            nullptr, (const bf16_t*)w, bias, bias_f32, (bf16_t*)out, 1, N, K, K, ldo, 0, 0, 0, 0, ra, na);
    TL_CHECK_LAUNCH("gemm_rope_normed");
    return TL_OK;
}

// tl_gemm_swiglu for one row whose x is the norm of the residual stream, made inside the kernel.  Returns
// TL_NOT_FUSED (nothing launched) for shapes it is not built for.
extern "C" int tl_gemm_swiglu_normed(const void* residual, void* residual_out, const void* pending, int parts, long part_stride,
                                     const void* norm_weight, int norm_weight_f32, float eps,
                                     const void* w, void* out, int I, int K, hipStream_t stream) {
    TL_REQUIRE(I > 0 && K > 0, "gemm_swiglu_normed: bad sizes I=%d K=%d", I, K);
    const NormArgs na = norm_args(residual, residual_out, pending, parts, part_stride, norm_weight, norm_weight_f32, eps);
    const int N = ((I + 31) / 32) * 64;          // rows of the interleaved matrix
    if (!norm_fits(na, K, 16 * 64) || ((uintptr_t)w % 16) || K / 64 / 16 >= 16)
        return TL_NOT_FUSED;
    const StripPlan p = plan_strips(I, 2 * TL_COMPUTE_UNITS, 16, false);       // every work-group makes x once and walks its run of outputs
    const size_t lds = (size_t)16 * 1024 + (size_t)(K + 8) * 2;
    gemm_skinny_kernel<1, 1, 16, bf16_t, true, true, 2, false, true><<<dim3(p.groups), dim3(16 * 64), lds, stream>>>(
        nullptr, (const bf16_t*)w, nullptr, 0, (bf16_t*)out, 1, N, K, K, I, I, 0, p.per_strip, p.per_group, RopeArgs{}, na);
    TL_CHECK_LAUNCH("gemm_swiglu_normed");
    return TL_OK;
}

// out[M, I] = silu(x g^T) * (x u^T) for bfloat16, with w = the gate and up matrices interleaved
// in blocks of 32 rows (rows 64 b .. 64 b + 31: gate rows 32 b .., rows 64 b + 32 ..: the up rows
// of the same columns), padded with zero rows to a multiple of 64.  The gate is applied to the
// float accumulators, as the reference's fused kernel does
// (/root/reference/src/torchlet/v10_triton_paged_gqa/kernel/ffn_swiglu.py:139-160).
extern "C" int tl_gemm_swiglu(const void* x, const void* w, void* out, int M, int I, int K, int ldx, int ldo,
                              hipStream_t stream) {
    TL_REQUIRE(M >= 0 && I > 0 && K > 0 && ldx >= K && ldo >= I, "gemm_swiglu: bad sizes M=%d I=%d K=%d", M, I, K);
    TL_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
               "gemm_swiglu: needs K and the row stride of x to be multiples of 8 and 16-byte aligned operands");
    if (M == 0) return TL_OK;
    const int N = ((I + 31) / 32) * 64;          // rows of the interleaved matrix
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    bf16_t* ob = (bf16_t*)out;
    // the few-rows kernel where its copy of x fits shared memory (else every wave fetches x as often
    // as its weights: 32B sizes, 16 rows, 20.2 against 18.9 ms a step)
    const bool x_fits = M == 1 || (size_t)16 * 1024 + (size_t)M * (K + 8) * 2 <= 156 * 1024;
    if ((M <= 16 && (x_fits || K % 64 != 0)) || (M <= 32 && K % 64 != 0)) {
        if (M <= 16) launch_skinny_t<1, 1, 16, bf16_t, true>(xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream);
        else launch_skinny_t<1, 2, 16, bf16_t, true>(xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream);
    } else if (K % 64 == 0) {
        const int rc = launch_dl_tile<bf16_t, true>(pick_dl_tile(M, N, K, true), xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream);
        if (rc != TL_OK) return rc;
    } else {
        int rc;
        switch (pick_tile(M, N)) {
        case TILE_256x256: rc = launch_mfma_tile_t<256, 256, 4, 2, bf16_t, true, 64>(xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream); break;
        case TILE_128x128_K32: rc = launch_mfma_tile_t<128, 128, 2, 2, bf16_t, true, 32>(xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream); break;
        case TILE_128x128_K64: rc = launch_mfma_tile_t<128, 128, 2, 2, bf16_t, true, 64>(xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream); break;
        default: rc = launch_mfma_tile_t<64, 128, 2, 2, bf16_t, true, 64>(xb, wb, nullptr, 0, ob, M, N, K, ldx, ldo, I, stream); break;
        }
        if (rc != TL_OK) return rc;
    }
    TL_CHECK_LAUNCH("gemm_swiglu");
    return TL_OK;
}

// out[P, M, N] (float) = partial sums of x w^T over P ranges of K, for a product with too few output
// tiles to fill the GPU (a narrow matrix against few rows): P work-groups per tile keep all compute
// units busy; whoever reads the slabs adds them up.  Returns P through `parts` (the caller sizes
// `out` for tl_gemm_partials_max()).  More than 64 rows: see plan_dl_split (measured at 512 rows:
// 3584 x 18944 147 -> 82 us, 5120 x 13824 179 -> 82 us, 5120 x 27648 348 -> 150 us, the norm's sum
// included).  Up to 64 rows, where it pays (see partials_on_tiles), the direct-load tile
// kernel runs with 64 x 64 tiles (measured at 64 rows, 3584 x 18944: 31 us with four parts against
// 90 us whole; 3584 x 3584: 9.5 against 20 us); for other K the skinny kernel
// with R = 4 strips per work-group, which share every x fetch.
extern "C" int tl_gemm_partials_max() { return 8; }

// Whether the tile kernel does the split: from 2 rows on, and for one row where the few-rows kernel
// has more than 256 strips of 16 weight rows to deal out.  Measured with the consumer's sum left out
// (us, few-rows kernel against split tiles): 3584 x 3584: 1 row 7.0 / 7.4, 2 rows 8.0 / 7.4, 8 rows 9.1 / 7.5,
// 16 rows 10.6 / 7.6; 5120 x 5120: 1 row 16.2 / 13.2, 8 rows 19.0 / 12.7, 16 rows 22.5 / 13.1;
// 3584 x 18944: 1 row 28.2 / 27.2, 8 rows 31.6 / 26.1, 16 rows 38.2 / 26.6; 5120 x 27648, one row: 70.8 / 53
// (320 strips, one work-group of eight waves with eight steps in flight per compute unit: two rounds,
// the second nearly empty).
static bool partials_on_tiles(int M, int N, int K) {
    return K % 64 == 0 && (M >= 2 || N > 16 * TL_COMPUTE_UNITS);
}

// Whether a consumer that can add slabs up should ask for them instead of the whole product.
extern "C" int tl_gemm_partials_pay(int M, int N, int K);

// How many parts tl_gemm_partials would use.
extern "C" int tl_gemm_partials_parts(int M, int N, int K) {
    if (M > 64 && K % 64 == 0) return plan_dl_split(M, N, K).parts;
    if (partials_on_tiles(M, N, K)) {
        const long tiles = (long)((M + 63) / 64) * ((N + 63) / 64);
        int P = (int)(TL_COMPUTE_UNITS / tiles);          // about one work-group per compute unit
        const int by_k = K / 512;                         // at least eight slabs of 64 per part
        if (P > by_k) P = by_k;
        if (P > 8) P = 8;
        return P < 1 ? 1 : P;
    }
    int P = (K + 63) / 64 / 32;                           // skinny kernel: at least 32 steps (2048 columns) per part
    if (P > 8) P = 8;
    return P < 1 ? 1 : P;
}

extern "C" int tl_gemm_partials_pay(int M, int N, int K) {
    return partials_on_tiles(M, N, K) && tl_gemm_partials_parts(M, N, K) > 1;
}

extern "C" int tl_gemm_partials(const void* x, const void* w, void* out, int M, int N, int K, int ldx, int* parts,
                                hipStream_t stream) {
    TL_REQUIRE(M > 0 && N > 0 && K > 0 && ldx >= K, "gemm_partials: bad sizes M=%d N=%d K=%d", M, N, K);
    TL_REQUIRE(K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
               "gemm_partials: needs K and the row stride of x to be multiples of 8 and 16-byte aligned operands");
    if (M > 64 && K % 64 == 0) {
        const DlSplit plan = plan_dl_split(M, N, K);
        *parts = plan.parts;
        const int rc = launch_dl_tile<float, false>(plan.tile, x, w, nullptr, 0, out, M, N, K, ldx, N, 0, stream, plan.parts, plan.k_per);
        if (rc != TL_OK) return rc;
        TL_CHECK_LAUNCH("gemm_partials");
        return TL_OK;
    }
    const int steps = (K + 63) / 64;
    int P = tl_gemm_partials_parts(M, N, K);
    const int k_per = ((steps + P - 1) / P) * 64;
    P = (K + k_per - 1) / k_per;
    *parts = P;
    if (partials_on_tiles(M, N, K)) {
        auto kernel = gemm_dl_tile_kernel<64, 64, 2, 2, 4, float, false>;
        constexpr size_t lds = (size_t)4 * 128 * 64 * sizeof(bf16_t);
        static hipError_t allowed = allow_lds(kernel, lds);
        TL_REQUIRE(allowed == hipSuccess, "gemm_partials: cannot get %zu bytes of shared memory", lds);
        dim3 grid(((M + 63) / 64) * ((N + 63) / 64), P), block(256);
        kernel<<<grid, block, lds, stream>>>((const bf16_t*)x, (const bf16_t*)w, nullptr, 0, (float*)out, M, N, K, ldx, N, 0, k_per);
        TL_CHECK_LAUNCH("gemm_partials");
        return TL_OK;
    }
    TL_REQUIRE(M <= 64, "gemm_partials: more than 64 rows need K to be a multiple of 64 (M=%d K=%d)", M, K);
    dim3 grid((N + 63) / 64, P), block(8 * 64);
    const size_t red_bytes = (size_t)8 * 4 * (M <= 16 ? 1 : (M <= 32 ? 2 : 4)) * 1024;
    if (M <= 16)
        gemm_skinny_kernel<4, 1, 8, float, false, false, skinny_depth<4, 1, 8>()><<<grid, block, red_bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, nullptr, 0, (float*)out, M, N, K, ldx, N, 0, k_per, 0, 0, RopeArgs{}, NormArgs{});
    else if (M <= 32)
        gemm_skinny_kernel<4, 2, 8, float, false, false, skinny_depth<4, 2, 8>()><<<grid, block, red_bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, nullptr, 0, (float*)out, M, N, K, ldx, N, 0, k_per, 0, 0, RopeArgs{}, NormArgs{});
    else {
        auto kernel = gemm_skinny_kernel<4, 4, 8, float, false, false, skinny_depth<4, 4, 8>()>;
        static hipError_t allowed = allow_lds(kernel, 128 * 1024);
        TL_REQUIRE(allowed == hipSuccess, "gemm_partials: cannot get %zu bytes of shared memory", red_bytes);
        kernel<<<grid, block, red_bytes, stream>>>((const bf16_t*)x, (const bf16_t*)w, nullptr, 0, (float*)out, M, N, K, ldx, N, 0, k_per, 0, 0, RopeArgs{}, NormArgs{});
    }
    TL_CHECK_LAUNCH("gemm_partials");
    return TL_OK;
}
