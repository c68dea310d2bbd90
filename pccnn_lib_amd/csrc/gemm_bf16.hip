// bf16 x bf16 -> fp32 GEMM on the CDNA4 matrix cores (v_mfma_f32_32x32x16_bf16), the contraction of the
// convolutions when their operands are kept in bf16 (fp32 accumulation, fp32 result).
//
// Workgroup tile 128 x 128 or 64 x 128 (4 wavefronts), inner step 32.  Whatever the operands' layout in memory,
// a tile sits in LDS as rows of k-pairs: dword [kp][x] = (element (x, 2kp), element (x, 2kp + 1)).  An operand
// whose reduction index is contiguous in memory already has its pairs packed and is scattered one dword per
// k-pair; an operand stored reduction-index-major is read two rows at a time and the rows are interleaved in
// registers.  Either way a fragment of the 32x32x16 MFMA (8 consecutive k of one row) is four conflict-free
// 32-bit LDS reads.  Tiles are double-buffered, global loads run two tiles ahead, one barrier per step; the
// tile order is XCD-aware and split-K partials are summed in a fixed order, as in the fp32 kernel.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define BG_N 128
#define BG_K 32            // bf16 elements of the reduction per step
#define BG_KP (BG_K / 2)   // k-pairs per step
#define BG_LD 132          // dwords per k-pair row (16-byte aligned rows)
#define BG_XCDS 8

struct GemmBf16Args {
    const uint16_t *a, *b;
    float *c;
    int64_t rows, cols, inner;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;
    int split_k;
    int64_t k_chunk;       // inner elements per split (multiple of BG_K)
    int aligned;           // pointers, leading dimensions and batch strides allow 16-byte loads
    int whole_units;       // aligned, and no 16-byte unit of a tile straddles the edge of its operand
    int tiles_x, tiles_y;
    int64_t total_wg;
};

// Global -> registers for one TILE_X x 32 operand tile.  MODE 1: 16-byte loads, nothing checked (tile inside the
// operand); MODE 2: 16-byte loads, a unit outside the operand reads as zeros (units are never cut: the host checks
// that the operand's extents along the units are multiples of 8); MODE 0: element by element.
// KCONTIG (element (x, k) at p[x * ld + k]): unit u = (x = u / 4, 8 consecutive k); TILE_X / 64 units per thread.
// otherwise (element (x, k) at p[k * ld + x]): unit u = (k-pair u / (TILE_X / 8), 8 consecutive x), both rows of
// the pair; one unit per thread, threads beyond the tile idle.
template <bool KCONTIG, int MODE, int TILE_X>
__device__ __forceinline__ void bg_tile_load(const uint16_t *__restrict__ p, int64_t ld, int64_t x0, int64_t x_end,
                                             int64_t k0, int64_t k_end, uint4 (&r)[2])
{
    if (KCONTIG) {
#pragma unroll
        for (int i = 0; i < TILE_X / 64; ++i) {
            const int u = threadIdx.x + 256 * i;
            const int64_t x = x0 + u / 4, k = k0 + (u % 4) * 8;
            if (MODE == 1) {
                r[i] = *(const uint4 *)(p + x * ld + k);
            } else if (MODE == 2) {
                r[i] = make_uint4(0, 0, 0, 0);
                if (x < x_end && k < k_end) r[i] = *(const uint4 *)(p + x * ld + k);
            } else {
                uint16_t v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = (x < x_end && k + e < k_end) ? p[x * ld + k + e] : (uint16_t)0;
                r[i] = make_uint4(v[0] | ((uint32_t)v[1] << 16), v[2] | ((uint32_t)v[3] << 16),
                                  v[4] | ((uint32_t)v[5] << 16), v[6] | ((uint32_t)v[7] << 16));
            }
        }
    } else {
        const int u = threadIdx.x;
        if (u < BG_KP * (TILE_X / 8)) {
            const int64_t k = k0 + 2 * (u / (TILE_X / 8)), x = x0 + (u % (TILE_X / 8)) * 8;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (MODE == 1) {
                    r[h] = *(const uint4 *)(p + (k + h) * ld + x);
                } else if (MODE == 2) {
                    r[h] = make_uint4(0, 0, 0, 0);
                    if (x < x_end && k + h < k_end) r[h] = *(const uint4 *)(p + (k + h) * ld + x);
                } else {
                    uint16_t v[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        v[e] = (x + e < x_end && k + h < k_end) ? p[(k + h) * ld + x + e] : (uint16_t)0;
                    r[h] = make_uint4(v[0] | ((uint32_t)v[1] << 16), v[2] | ((uint32_t)v[3] << 16),
                                      v[4] | ((uint32_t)v[5] << 16), v[6] | ((uint32_t)v[7] << 16));
                }
            }
        }
    }
}

template <bool KCONTIG, int TILE_X>
__device__ __forceinline__ void bg_tile_store(uint32_t (*lds)[BG_LD], const uint4 (&r)[2])
{
    if (KCONTIG) {
#pragma unroll
        for (int i = 0; i < TILE_X / 64; ++i) {
            const int u = threadIdx.x + 256 * i;
            const int x = u / 4, kp = (u % 4) * 4;
            lds[kp + 0][x] = r[i].x;
            lds[kp + 1][x] = r[i].y;
            lds[kp + 2][x] = r[i].z;
            lds[kp + 3][x] = r[i].w;
        }
    } else {
        const int u = threadIdx.x;
        if (u < BG_KP * (TILE_X / 8)) {
            const int kp = u / (TILE_X / 8), x = (u % (TILE_X / 8)) * 8;
            const uint32_t lo[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
            const uint32_t hi[4] = {r[1].x, r[1].y, r[1].z, r[1].w};
            uint32_t o[8];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                o[2 * q] = (lo[q] & 0xffffu) | (hi[q] << 16);
                o[2 * q + 1] = (lo[q] >> 16) | (hi[q] & 0xffff0000u);
            }
            *(uint4 *)&lds[kp][x] = make_uint4(o[0], o[1], o[2], o[3]);
            *(uint4 *)&lds[kp][x + 4] = make_uint4(o[4], o[5], o[6], o[7]);
        }
    }
}

template <bool AT, bool BT, int MODE, int BM>
__device__ __forceinline__ void bg_tile_loop(const GemmBf16Args &g, const uint16_t *__restrict__ a,
                                             const uint16_t *__restrict__ b, int64_t bm, int64_t bn, int64_t k_begin,
                                             int64_t k_end, uint32_t (*As)[BG_KP][BG_LD], uint32_t (*Bs)[BG_KP][BG_LD],
                                             floatx16 (&acc)[2][BM / 64])
{
    constexpr int WN = 4 / (BM / 64);                               // wavefronts along the columns
    constexpr int TN = BM / 64;                                     // 32-column MFMA tiles per wavefront
    const int lane = pccnn_lane();
    const int wave = threadIdx.x >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int frag_g = lane >> 5, frag_c = lane & 31;
    uint4 ra[2], rb[2];
    const int64_t nk = (k_end - k_begin + BG_K - 1) / BG_K;
    // A stored [rows, inner] (AT = false) and B stored [cols, inner] (BT = true) have the reduction index contiguous.
    if (nk > 0) {
        bg_tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k_begin, k_end, ra);
        bg_tile_load<BT, MODE, BG_N>(b, g.ldb, bn, g.cols, k_begin, k_end, rb);
        bg_tile_store<!AT, BM>(As[0], ra);
        bg_tile_store<BT, BG_N>(Bs[0], rb);
    }
    if (nk > 1) {
        bg_tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k_begin + BG_K, k_end, ra);
        bg_tile_load<BT, MODE, BG_N>(b, g.ldb, bn, g.cols, k_begin + BG_K, k_end, rb);
    }
    __syncthreads();
    for (int64_t kt = 0; kt < nk; ++kt) {
        const int buf = (int)(kt & 1);
#pragma unroll
        for (int ks = 0; ks < BG_K / 16; ++ks) {
            // lanes 0..31 hold k = 16 ks + 0..7 of their row, lanes 32..63 hold k = 16 ks + 8..15: four k-pairs each
            const int kp = 8 * ks + 4 * frag_g;
            uint4 fa[2], fb[TN];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int x = wm * 64 + i * 32 + frag_c;
                fa[i] = make_uint4(As[buf][kp][x], As[buf][kp + 1][x], As[buf][kp + 2][x], As[buf][kp + 3][x]);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int x = wn * (32 * TN) + j * 32 + frag_c;
                fb[j] = make_uint4(Bs[buf][kp][x], Bs[buf][kp + 1][x], Bs[buf][kp + 2][x], Bs[buf][kp + 3][x]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[i]),
                                                                        __builtin_bit_cast(bf16x8, fb[j]), acc[i][j],
                                                                        0, 0, 0);
            if (ks == 0) {
                // tile kt+1 (in registers since the previous step) goes to the free LDS buffer, and the
                // registers take the loads of tile kt+2
                if (kt + 1 < nk) {
                    bg_tile_store<!AT, BM>(As[buf ^ 1], ra);
                    bg_tile_store<BT, BG_N>(Bs[buf ^ 1], rb);
                }
                if (kt + 2 < nk) {
                    const int64_t k0 = k_begin + (kt + 2) * BG_K;
                    bg_tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k0, k_end, ra);
                    bg_tile_load<BT, MODE, BG_N>(b, g.ldb, bn, g.cols, k0, k_end, rb);
                }
            }
        }
        __syncthreads();
    }
}

template <bool AT, bool BT, int BM>
__global__ void __launch_bounds__(256)
gemm_bf16_mfma_kernel(GemmBf16Args g, float *__restrict__ partial)
{
    __shared__ __attribute__((aligned(16))) uint32_t As[2][BG_KP][BG_LD];
    __shared__ __attribute__((aligned(16))) uint32_t Bs[2][BG_KP][BG_LD];
    constexpr int WN = 4 / (BM / 64);
    constexpr int TN = BM / 64;

    const int lane = pccnn_lane();
    const int wave = threadIdx.x >> 6;
    const int wm = wave / WN, wn = wave % WN;
    // every XCD (workgroups are dealt to the 8 XCDs round-robin) owns one contiguous run of logical tiles
    const int64_t per_xcd = (int64_t)gridDim.x / BG_XCDS;
    const int64_t tile = (int64_t)(blockIdx.x % BG_XCDS) * per_xcd + blockIdx.x / BG_XCDS;
    if (tile >= g.total_wg) return;                                 // padding of the launch
    const int tx = (int)(tile % g.tiles_x);
    const int ty = (int)((tile / g.tiles_x) % g.tiles_y);
    const int tz = (int)(tile / ((int64_t)g.tiles_x * g.tiles_y));
    const int batch = tz / g.split_k;
    const int split = tz % g.split_k;
    const int64_t bm = (int64_t)ty * BM;
    const int64_t bn = (int64_t)tx * BG_N;
    const uint16_t *a = g.a + (int64_t)batch * g.stride_a;
    const uint16_t *b = g.b + (int64_t)batch * g.stride_b;
    const int64_t k_begin = (int64_t)split * g.k_chunk;
    const int64_t k_end = (k_begin + g.k_chunk < g.inner) ? k_begin + g.k_chunk : g.inner;
    const bool fast = g.aligned && (bm + BM <= g.rows) && (bn + BG_N <= g.cols) && ((k_end - k_begin) % BG_K == 0);

    floatx16 acc[2][TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    if (fast) bg_tile_loop<AT, BT, 1, BM>(g, a, b, bm, bn, k_begin, k_end, As, Bs, acc);
    else if (g.whole_units) bg_tile_loop<AT, BT, 2, BM>(g, a, b, bm, bn, k_begin, k_end, As, Bs, acc);
    else bg_tile_loop<AT, BT, 0, BM>(g, a, b, bm, bn, k_begin, k_end, As, Bs, acc);

    // Accumulator layout of the 32x32 MFMA: register v of lane l holds
    // row 8*(v/4) + 4*(l/32) + v%4, column l%32 of the tile.
    float *cbase;
    int64_t ldc;
    if (g.split_k > 1) {
        cbase = partial + ((int64_t)batch * g.split_k + split) * g.rows * g.cols;
        ldc = g.cols;
    } else {
        cbase = g.c + (int64_t)batch * g.stride_c;
        ldc = g.ldc;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int64_t col = bn + wn * (32 * TN) + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int64_t row = bm + wm * 64 + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (row < g.rows && col < g.cols) cbase[row * ldc + col] = acc[i][j][v];
            }
        }
}

__global__ void __launch_bounds__(256)
bg_splitk_reduce_kernel(const float *__restrict__ partial, GemmBf16Args g, int batch_count)
{
    const int64_t per = g.rows * g.cols;
    const int64_t total = per * batch_count;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t bi = i / per, e = i % per;
        const float *src = partial + bi * g.split_k * per + e;
        float s = 0.0f;
        int k = 0;
        for (; k + 8 <= g.split_k; k += 8) {                        // eight loads in flight, added in order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(int64_t)(k + u) * per];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; k < g.split_k; ++k) s += src[(int64_t)k * per];
        g.c[bi * g.stride_c + (e / g.cols) * g.ldc + (e % g.cols)] = s;
    }
}

// fp32 -> bf16, round to nearest even (NaN stays NaN).
__global__ void __launch_bounds__(256)
f32_to_bf16_kernel(const float *__restrict__ src, uint16_t *__restrict__ dst, int64_t count)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (int64_t)gridDim.x * blockDim.x)
        dst[i] = pccnn_bf16_bits(src[i]);
}

extern "C" int pccnn_f32_to_bf16(const float *src, uint16_t *dst, int64_t count, void *stream)
{
    PCCNN_REQUIRE(count >= 0, PCCNN_ERR_INVALID, "pccnn_f32_to_bf16: count=%lld", (long long)count);
    if (count == 0) return PCCNN_OK;
    PCCNN_REQUIRE(src && dst, PCCNN_ERR_INVALID, "pccnn_f32_to_bf16: null pointer");
    int64_t blocks = pccnn_ceil_div(count, 256);
    if (blocks > 8192) blocks = 8192;
    f32_to_bf16_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(src, dst, count);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" int pccnn_gemm_bf16(const uint16_t *a, const uint16_t *b, float *c, int64_t rows, int64_t cols,
                               int64_t inner, int a_trans, int b_trans, int64_t lda, int64_t ldb, int64_t ldc,
                               int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, int split_k,
                               void *workspace, size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(rows >= 0 && cols >= 0 && inner >= 0 && batch >= 1, PCCNN_ERR_INVALID,
                  "pccnn_gemm_bf16: rows=%lld cols=%lld inner=%lld batch=%d", (long long)rows, (long long)cols,
                  (long long)inner, batch);
    if (rows == 0 || cols == 0) return PCCNN_OK;
    PCCNN_REQUIRE(a && b && c, PCCNN_ERR_INVALID, "pccnn_gemm_bf16: null pointer");
    PCCNN_REQUIRE(lda >= (a_trans ? rows : inner) && ldb >= (b_trans ? inner : cols) && ldc >= cols, PCCNN_ERR_INVALID,
                  "pccnn_gemm_bf16: leading dimension too small (lda=%lld ldb=%lld ldc=%lld)", (long long)lda,
                  (long long)ldb, (long long)ldc);
    if (split_k < 1) split_k = 1;
    GemmBf16Args g;
    g.a = a; g.b = b; g.c = c;
    g.rows = rows; g.cols = cols; g.inner = inner;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.stride_a = stride_a; g.stride_b = stride_b; g.stride_c = stride_c;
    int64_t chunk = pccnn_ceil_div(pccnn_ceil_div(inner > 0 ? inner : 1, split_k), BG_K) * BG_K;
    split_k = (int)pccnn_ceil_div(inner > 0 ? inner : 1, chunk);
    g.split_k = split_k;
    g.k_chunk = chunk;
    g.aligned = ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0) && (lda % 8 == 0) && (ldb % 8 == 0) &&
                (stride_a % 8 == 0) && (stride_b % 8 == 0);
    // units run along the reduction index where that is contiguous in memory, else along the rows / columns
    g.whole_units = g.aligned && ((a_trans ? rows : inner) % 8 == 0) && ((b_trans ? inner : cols) % 8 == 0);
    float *partial = nullptr;
    if (split_k > 1) {
        size_t need = (size_t)batch * split_k * rows * cols * sizeof(float);
        PCCNN_REQUIRE(workspace && workspace_bytes >= need, PCCNN_ERR_WORKSPACE,
                      "pccnn_gemm_bf16: split-k workspace of %zu bytes, need %zu", workspace_bytes, need);
        partial = (float *)workspace;
    }
    hipStream_t s = (hipStream_t)stream;
    // 128-row tiles unless that leaves the chip short of workgroups: then 64-row tiles
    const int64_t wg128 = pccnn_ceil_div(cols, BG_N) * pccnn_ceil_div(rows, 128) * batch * split_k;
    const int bm_tile = wg128 >= 1024 ? 128 : 64;
    g.tiles_x = (int)pccnn_ceil_div(cols, BG_N);
    g.tiles_y = (int)pccnn_ceil_div(rows, bm_tile);
    g.total_wg = (int64_t)g.tiles_x * g.tiles_y * batch * split_k;
    PCCNN_REQUIRE(g.total_wg < (1ll << 31) - BG_XCDS, PCCNN_ERR_UNSUPPORTED, "pccnn_gemm_bf16: grid too large");
    dim3 grid((unsigned)(pccnn_ceil_div(g.total_wg, BG_XCDS) * BG_XCDS));
    {
        PccnnTimed timed(PCCNN_T_GEMM, s);
#define GEMM_GO(AT, BT)                                                                        \
    do {                                                                                       \
        if (bm_tile == 128) gemm_bf16_mfma_kernel<AT, BT, 128><<<grid, 256, 0, s>>>(g, partial); \
        else gemm_bf16_mfma_kernel<AT, BT, 64><<<grid, 256, 0, s>>>(g, partial);                 \
    } while (0)
        if (!a_trans && !b_trans) GEMM_GO(false, false);
        else if (!a_trans && b_trans) GEMM_GO(false, true);
        else if (a_trans && !b_trans) GEMM_GO(true, false);
        else GEMM_GO(true, true);
#undef GEMM_GO
    }
    PCCNN_LAUNCH_CHECK();
    if (split_k > 1) {
        int64_t total = rows * cols * batch;
        int64_t blocks = pccnn_ceil_div(total, 256);
        if (blocks > 4096) blocks = 4096;
        bg_splitk_reduce_kernel<<<(unsigned)blocks, 256, 0, s>>>(partial, g, batch);
        PCCNN_LAUNCH_CHECK();
    }
    return PCCNN_OK;
}
