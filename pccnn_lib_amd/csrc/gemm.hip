// fp32 GEMM on the CDNA matrix cores (v_mfma_f32_32x32x2_f32), used for the
// [M, K*Cin] x [K*Cin, Cout] contraction of the convolutions and its two transposes.
//
// Two kernels.  gemm_f32_full_tiles_kernel takes the products whose tiles are all full (the shapes of the
// convolutions: thousands of rows, a multiple of 128 columns): its k loop holds nothing but MFMAs, four or three
// 16-byte global loads, as many 16-byte LDS stores and the fragment reads.  gemm_f32_mfma_kernel takes everything
// else (edge tiles, odd leading dimensions, very short reductions) with bounds checks where a tile needs them.
//
// Common to both: workgroup tile 128 x 128 (4 wavefronts as 2 x 2, each a 64 x 64 block of 2 x 2 MFMA tiles) or,
// when the grid would otherwise be too small to fill the chip, 64 x 128 (1 x 4 wavefronts of 64 x 32); inner step
// 16; operand tiles double-buffered in LDS, the next tile's global loads issued before the current tile's MFMAs,
// one barrier per step.  Split-K writes partial products to a workspace that a second kernel sums in a fixed order.
#include <type_traits>

#include "common.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define GT_M 128
#define GT_N 128
#define GT_K 16
#define GT_LD 130          // LDS row stride (floats): conflict-free transposing stores, 8-byte aligned rows

struct GemmArgs {
    const float *a, *b;
    float *c;
    int64_t rows, cols, inner;
    int64_t lda, ldb, ldc;
    int64_t stride_a, stride_b, stride_c;
    int split_k;
    int64_t k_chunk;       // inner elements per split (multiple of GT_K)
    int aligned;           // pointers, leading dimensions and batch strides allow float4 loads
    int whole_units;       // aligned, and no float4 unit of a tile straddles the edge of its operand
    int tiles_x, tiles_y;  // workgroup tiles along the columns / rows
    int64_t total_wg;      // tiles_x * tiles_y * batch * split_k
};

// Workgroups are handed to the 8 XCDs round-robin by their linear id, and each XCD has its own L2.  The
// launch is one-dimensional and padded to a multiple of 8; workgroup i works on logical tile
// (i % 8) * (padded / 8) + i / 8, so every XCD owns one contiguous run of logical tiles.  Logical tiles are
// ordered column tile fastest, then row tile, then batch / split: neighbours in that order share their A
// row tile (or, with one column tile, their B chunk), which is then fetched from HBM by one XCD, once.
#define GEMM_XCDS 8

// Global -> registers for one 128 x 16 operand tile.  `KCONTIG`: the reduction index is the
// contiguous one in memory (element (x, k) at p[x * ld + k]); otherwise element (x, k) at p[k * ld + x].
// MODE 1: the tile is fully inside the matrix and 16-byte aligned, so it is read with float4 loads and no checks;
// MODE 2: float4 loads, a unit outside the matrix reads as zeros (the host checks that no unit straddles an edge:
// the extents along the units are multiples of 4); MODE 0: element by element.
template <bool KCONTIG, int MODE, int TILE_X>
__device__ __forceinline__ void tile_load(const float *__restrict__ p, int64_t ld, int64_t x0, int64_t x_end,
                                          int64_t k0, int64_t k_end, float4 (&r)[TILE_X / 64 * (GT_K / 16)])
{
#pragma unroll
    for (int i = 0; i < TILE_X / 64 * (GT_K / 16); ++i) {
        const int idx = threadIdx.x + 256 * i;
        int64_t x, k;
        if (KCONTIG) { x = x0 + idx / (GT_K / 4); k = k0 + (idx % (GT_K / 4)) * 4; }
        else { k = k0 + idx / (TILE_X / 4); x = x0 + (idx % (TILE_X / 4)) * 4; }
        if (MODE == 1) {
            r[i] = KCONTIG ? *(const float4 *)(p + x * ld + k) : *(const float4 *)(p + k * ld + x);
        } else if (MODE == 2) {
            r[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (x < x_end && k < k_end)
                r[i] = KCONTIG ? *(const float4 *)(p + x * ld + k) : *(const float4 *)(p + k * ld + x);
        } else {
            float v[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int64_t xx = KCONTIG ? x : x + c;
                const int64_t kk = KCONTIG ? k + c : k;
                v[c] = (xx < x_end && kk < k_end) ? (KCONTIG ? p[xx * ld + kk] : p[kk * ld + xx]) : 0.0f;
            }
            r[i] = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
}

template <bool KCONTIG, int TILE_X>
__device__ __forceinline__ void tile_store(float (*lds)[GT_LD], const float4 (&r)[TILE_X / 64 * (GT_K / 16)])
{
#pragma unroll
    for (int i = 0; i < TILE_X / 64 * (GT_K / 16); ++i) {
        const int idx = threadIdx.x + 256 * i;
        if (KCONTIG) {
            const int x = idx / (GT_K / 4), k = (idx % (GT_K / 4)) * 4;
            lds[k + 0][x] = r[i].x;
            lds[k + 1][x] = r[i].y;
            lds[k + 2][x] = r[i].z;
            lds[k + 3][x] = r[i].w;
        } else {
            const int k = idx / (TILE_X / 4), x = (idx % (TILE_X / 4)) * 4;
            *(float2 *)&lds[k][x] = make_float2(r[i].x, r[i].y);
            *(float2 *)&lds[k][x + 2] = make_float2(r[i].z, r[i].w);
        }
    }
}

// The k loop of one workgroup tile.  Global loads run two or three tiles ahead of the MFMAs (one or two register
// sets, then the free LDS buffer); inside a tile the LDS fragments of sub-step ks+1 are read before the MFMAs of
// sub-step ks are issued, so the matrix pipe never waits on an LDS round trip.
template <bool AT, bool BT, int MODE, int BM>
__device__ __forceinline__ void gemm_tile_loop(const GemmArgs &g, const float *__restrict__ a,
                                               const float *__restrict__ b, int64_t bm, int64_t bn, int64_t k_begin,
                                               int64_t k_end, float (*As)[GT_K][GT_LD], float (*Bs)[GT_K][GT_LD],
                                               floatx16 (&acc)[2][BM / 64])
{
    constexpr int WN = 4 / (BM / 64);                               // wavefronts along the columns
    constexpr int TN = BM / 64;                                     // 32-column MFMA tiles per wavefront
    const int lane = pccnn_lane();
    const int wave = threadIdx.x >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int frag_k = lane >> 5, frag_c = lane & 31;
    constexpr int NA = BM / 64 * (GT_K / 16), NB = 2 * (GT_K / 16);
    // 64-row tiles on the fast path travel in two register sets (tile j in set j & 1), so every global load has
    // two whole steps of MFMAs to arrive (3 - 4 % on the products of 65 536 x 1024 x 128).  The 128-row tiles keep
    // one set (AHEAD = 2): with two they pass 128 registers, which halves the waves per SIMD and costs 9 %; so does
    // the bounds-checked path of edge tiles.
    constexpr bool DEEP = MODE == 1 && BM == 64;
    constexpr int AHEAD = DEEP ? 3 : 2;
    float4 ra0[NA], rb0[NB], ra1[DEEP ? NA : 1], rb1[DEEP ? NB : 1];
    const int64_t nk = (k_end - k_begin + GT_K - 1) / GT_K;
    // A stored [rows, inner] (AT = false) has the reduction index contiguous; B stored
    // [inner, cols] (BT = false) has the column index contiguous.
    if (nk > 0) {
        tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k_begin, k_end, ra0);
        tile_load<BT, MODE, GT_N>(b, g.ldb, bn, g.cols, k_begin, k_end, rb0);
        tile_store<!AT, BM>(As[0], ra0);
        tile_store<BT, GT_N>(Bs[0], rb0);
    }
    if constexpr (DEEP) {
        if (nk > 1) {
            tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k_begin + GT_K, k_end, ra1);
            tile_load<BT, MODE, GT_N>(b, g.ldb, bn, g.cols, k_begin + GT_K, k_end, rb1);
        }
        if (nk > 2) {
            tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k_begin + 2 * GT_K, k_end, ra0);
            tile_load<BT, MODE, GT_N>(b, g.ldb, bn, g.cols, k_begin + 2 * GT_K, k_end, rb0);
        }
    } else if (nk > 1) {
        tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k_begin + GT_K, k_end, ra0);
        tile_load<BT, MODE, GT_N>(b, g.ldb, bn, g.cols, k_begin + GT_K, k_end, rb0);
    }
    __syncthreads();
    // One step: the MFMAs of tile kt from LDS buffer kt & 1.  Behind the first of them tile kt+1, which sits in
    // the register set (ra, rb), is parked in the other LDS buffer (free since the barrier that ended step kt-1)
    // and the same registers take the loads of tile kt+AHEAD.
    auto step = [&](int64_t kt, float4 (&ra)[NA], float4 (&rb)[NB]) {
        const int buf = (int)(kt & 1);
        float fa[2][2], fb[2][TN];
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[0][i] = As[buf][frag_k][wm * 64 + i * 32 + frag_c];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[0][j] = Bs[buf][frag_k][wn * (32 * TN) + j * 32 + frag_c];
#pragma unroll
        for (int ks = 0; ks < GT_K / 2; ++ks) {
            const int cur = ks & 1, nxt = cur ^ 1;
            if (ks + 1 < GT_K / 2) {
                const int kr = 2 * (ks + 1) + frag_k;
#pragma unroll
                for (int i = 0; i < 2; ++i) fa[nxt][i] = As[buf][kr][wm * 64 + i * 32 + frag_c];
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[nxt][j] = Bs[buf][kr][wn * (32 * TN) + j * 32 + frag_c];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
            if (ks == 0) {
                // behind the first MFMAs of the step, so the matrix pipe is busy while this wave moves data
                if (kt + 1 < nk) {
                    tile_store<!AT, BM>(As[buf ^ 1], ra);
                    tile_store<BT, GT_N>(Bs[buf ^ 1], rb);
                }
                if (kt + AHEAD < nk) {
                    const int64_t k0 = k_begin + (kt + AHEAD) * GT_K;
                    tile_load<!AT, MODE, BM>(a, g.lda, bm, g.rows, k0, k_end, ra);
                    tile_load<BT, MODE, GT_N>(b, g.ldb, bn, g.cols, k0, k_end, rb);
                }
            }
            // keep the order written above in the instruction stream: the fragment reads of the next sub-step go
            // out before this sub-step's MFMAs, so their LDS latency is covered by the matrix pipe
            if (ks + 1 < GT_K / 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2 * TN, 0);
        }
        __syncthreads();
    };
    if constexpr (DEEP) {
        for (int64_t kt = 0; kt < nk; kt += 2) {
            step(kt, ra1, rb1);                                     // tile kt+1 (odd) travels in set 1
            if (kt + 1 < nk) step(kt + 1, ra0, rb0);                // tile kt+2 (even) in set 0
        }
    } else {
        for (int64_t kt = 0; kt < nk; ++kt) step(kt, ra0, rb0);
    }
}

template <bool AT, bool BT, int BM>
__global__ void __launch_bounds__(256)
gemm_f32_mfma_kernel(GemmArgs g, float *__restrict__ partial)
{
    __shared__ __attribute__((aligned(16))) float As[2][GT_K][GT_LD];
    __shared__ __attribute__((aligned(16))) float Bs[2][GT_K][GT_LD];
    constexpr int WN = 4 / (BM / 64);
    constexpr int TN = BM / 64;

    const int lane = pccnn_lane();
    const int wave = threadIdx.x >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int64_t per_xcd = (int64_t)gridDim.x / GEMM_XCDS;
    const int64_t tile = (int64_t)(blockIdx.x % GEMM_XCDS) * per_xcd + blockIdx.x / GEMM_XCDS;
    if (tile >= g.total_wg) return;                                 // padding of the launch
    const int tx = (int)(tile % g.tiles_x);
    const int ty = (int)((tile / g.tiles_x) % g.tiles_y);
    const int tz = (int)(tile / ((int64_t)g.tiles_x * g.tiles_y));
    const int batch = tz / g.split_k;
    const int split = tz % g.split_k;
    const int64_t bm = (int64_t)ty * BM;
    const int64_t bn = (int64_t)tx * GT_N;
    const float *a = g.a + (int64_t)batch * g.stride_a;
    const float *b = g.b + (int64_t)batch * g.stride_b;
    const int64_t k_begin = (int64_t)split * g.k_chunk;
    const int64_t k_end = (k_begin + g.k_chunk < g.inner) ? k_begin + g.k_chunk : g.inner;
    const bool fast = g.aligned && (bm + BM <= g.rows) && (bn + GT_N <= g.cols) && ((k_end - k_begin) % GT_K == 0);

    floatx16 acc[2][TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    if (fast) gemm_tile_loop<AT, BT, 1, BM>(g, a, b, bm, bn, k_begin, k_end, As, Bs, acc);
    else if (g.whole_units) gemm_tile_loop<AT, BT, 2, BM>(g, a, b, bm, bn, k_begin, k_end, As, Bs, acc);
    else gemm_tile_loop<AT, BT, 0, BM>(g, a, b, bm, bn, k_begin, k_end, As, Bs, acc);

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

// ---------------------------------------------------------------------------------------------------------------
// The kernel for full tiles (rows % BM == 0, cols % 128 == 0, every k range a multiple of 16, 16-byte alignment).
// On this part vector-ALU and memory instructions are not hidden behind the MFMAs of the other wavefronts of a
// SIMD: a k step costs its MFMA cycles plus about 4 cycles per vector instruction and about 60 per global load.
// The loop therefore carries no address arithmetic at all:
//  * global loads take a uniform base (advanced with scalar adds) and a 32-bit lane offset computed once;
//  * the k loop is unrolled over the two LDS buffers, so every LDS address is a register plus an immediate;
//  * an operand whose reduction index is contiguous in memory ("KC": A [rows, inner], B [cols, inner]) keeps its
//    16-byte chunks (4 k) whole: one ds_write_b128 per chunk, and the lane that feeds row r of a 32-row MFMA tile
//    reads a whole chunk back (ds_read_b128).  Chunk c of row r sits in slot c ^ swz(r), so that the lanes of one
//    LDS pass hit distinct banks.  An operand whose row / column index is contiguous ("XC") lands k-major; the k
//    rows with (k >> 2) & 1 set are rotated by 32 elements so that the two halves of a wavefront, which read
//    different k, use different banks;
//  * which k a lane multiplies in which MFMA is free as long as both operands agree: lane half h takes
//    k = 4 (2 j + h) + e in the e-th MFMA of group j (e = 0..3, j = 0..1 per 16-k tile).
// One barrier per k step, in its middle: behind it the buffer of the current tile is free and the next tile is
// complete, whose first fragments are requested before the second half of the step's MFMAs.
__device__ __forceinline__ int gl_row_swz(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }

// byte offset, from the tile's origin, of the 16-byte chunk this lane loads first; its i-th load is the same lane
// offset from a base moved on by gl_load_delta() elements
template <bool KC, int X>
__device__ __forceinline__ unsigned gl_lane_offset(int wave, int lane, int64_t ld)
{
    const int q = wave * (X / 64);
    if (KC) {
        const int row = q * 16 + (lane >> 2);
        return (unsigned)((row * ld + (((lane & 3) ^ gl_row_swz(row)) << 2)) * 4);
    }
    const int e = q * 64 + lane;
    const int k = e / (X / 4), pos = e % (X / 4);
    return (unsigned)((k * ld + ((pos ^ (((k >> 2) & 1) << 3)) << 2)) * 4);
}
template <bool KC, int X>
__device__ __forceinline__ int64_t gl_load_delta(int64_t ld) { return KC ? 16 * ld : (256 / X) * ld; }

template <bool AT, bool BT, int BM>
__global__ void __launch_bounds__(256)
gemm_f32_full_tiles_kernel(GemmArgs g, float *__restrict__ partial)
{
    constexpr bool AKC = !AT, BKC = BT;
    constexpr int WN = 4 / (BM / 64);                               // wavefronts along the columns
    constexpr int TN = BM / 64;                                     // 32-column MFMA tiles per wavefront
    constexpr int NA = BM / 64, NB = GT_N / 64;                     // 16-byte loads per lane and k tile
    __shared__ __attribute__((aligned(16))) float As[2][BM * GT_K];
    __shared__ __attribute__((aligned(16))) float Bs[2][GT_N * GT_K];

    const int lane = pccnn_lane();
    const int wave = threadIdx.x >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int r = lane & 31, h = lane >> 5;
    const int64_t per_xcd = (int64_t)gridDim.x / GEMM_XCDS;
    const int64_t tile = (int64_t)(blockIdx.x % GEMM_XCDS) * per_xcd + blockIdx.x / GEMM_XCDS;
    if (tile >= g.total_wg) return;
    const int tx = (int)(tile % g.tiles_x);
    const int ty = (int)((tile / g.tiles_x) % g.tiles_y);
    const int tz = (int)(tile / ((int64_t)g.tiles_x * g.tiles_y));
    const int batch = tz / g.split_k;
    const int split = tz % g.split_k;
    const int64_t bm = (int64_t)ty * BM;
    const int64_t bn = (int64_t)tx * GT_N;
    const int64_t k_begin = (int64_t)split * g.k_chunk;
    const int64_t k_end = (k_begin + g.k_chunk < g.inner) ? k_begin + g.k_chunk : g.inner;
    const int64_t nk = (k_end - k_begin) / GT_K;
    // uniform: the origin of the current k tile of either operand
    const float *a_tile = g.a + (int64_t)batch * g.stride_a + (AKC ? bm * g.lda + k_begin : k_begin * g.lda + bm);
    const float *b_tile = g.b + (int64_t)batch * g.stride_b + (BKC ? bn * g.ldb + k_begin : k_begin * g.ldb + bn);
    const int64_t a_step = AKC ? GT_K : GT_K * g.lda;
    const int64_t b_step = BKC ? GT_K : GT_K * g.ldb;
    const unsigned a_lane = gl_lane_offset<AKC, BM>(wave, lane, g.lda);
    const unsigned b_lane = gl_lane_offset<BKC, GT_N>(wave, lane, g.ldb);
    const int64_t a_delta = gl_load_delta<AKC, BM>(g.lda), b_delta = gl_load_delta<BKC, GT_N>(g.ldb);

    floatx16 acc[2][TN];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // where this lane parks its loads (floats from the start of a buffer) and where its fragments are
    const int a_park = (wave * NA * 64 + lane) * 4, b_park = (wave * NB * 64 + lane) * 4;
    int a_off[2], b_off[TN];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int x = (BM == 64 ? 0 : wm * 64) + i * 32 + r;
        a_off[i] = AKC ? x * GT_K + ((h ^ gl_row_swz(r)) << 2) : (4 * h) * BM + (x ^ (h << 5));
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int x = wn * (32 * TN) + j * 32 + r;
        b_off[j] = BKC ? x * GT_K + ((h ^ gl_row_swz(r)) << 2) : (4 * h) * GT_N + (x ^ (h << 5));
    }

    // A tile is requested one k step before it is parked in LDS.  (Two register sets, two steps ahead, were
    // measured and are not faster.)
    floatx4 ra[NA], rb[NB];
    auto load_tile = [&]() __attribute__((always_inline)) {         // the tile at (a_tile, b_tile), which move on
#pragma unroll
        for (int i = 0; i < NA; ++i) ra[i] = *(const floatx4 *)((const char *)(a_tile + i * a_delta) + a_lane);
#pragma unroll
        for (int i = 0; i < NB; ++i) rb[i] = *(const floatx4 *)((const char *)(b_tile + i * b_delta) + b_lane);
        a_tile += a_step;
        b_tile += b_step;
    };
    auto park_tile = [&](float *as, float *bs) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NA; ++i) *(floatx4 *)(as + a_park + i * 256) = ra[i];
#pragma unroll
        for (int i = 0; i < NB; ++i) *(floatx4 *)(bs + b_park + i * 256) = rb[i];
    };
    float fa[2][2][4], fb[2][TN][4];                                // [half j of the tile][MFMA tile][e]
    auto read_frags = [&](const float *as, const float *bs, int j) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (AKC) {
                // chunk 2 j + h sits in slot (2 j + h) ^ swz = (h ^ swz) ^ 2 j
                const floatx4 v = *(const floatx4 *)(as + (a_off[i] ^ (j << 3)));
                fa[j][i][0] = v.x; fa[j][i][1] = v.y; fa[j][i][2] = v.z; fa[j][i][3] = v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) fa[j][i][e] = as[a_off[i] + (8 * j + e) * BM];
            }
        }
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            if (BKC) {
                const floatx4 v = *(const floatx4 *)(bs + (b_off[t] ^ (j << 3)));
                fb[j][t][0] = v.x; fb[j][t][1] = v.y; fb[j][t][2] = v.z; fb[j][t][3] = v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) fb[j][t][e] = bs[b_off[t] + (8 * j + e) * GT_N];
            }
        }
    };
    auto mfmas = [&](int j) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int t = 0; t < TN; ++t)
                    acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][t][e], fa[j][i][e], acc[i][t], 0, 0, 0);
    };
    // this wave's LDS traffic is complete, then everyone's (the global loads stay in flight)
    auto lds_barrier = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // One k tile, whose first half is in the registers on entry: `cur` is its buffer, `nxt` takes tile kt + 1
    // (in the registers since the previous step) before the barrier.
    auto step = [&](auto cur_c, int64_t kt, auto full) __attribute__((always_inline)) {
        constexpr int cur = decltype(cur_c)::value, nxt = cur ^ 1;
        read_frags(As[cur], Bs[cur], 1);
        __builtin_amdgcn_sched_barrier(0);
        mfmas(0);
        __builtin_amdgcn_sched_barrier(0);
        if (full || kt + 1 < nk) {
            park_tile(As[nxt], Bs[nxt]);
            lds_barrier();
            if (full || kt + 2 < nk) load_tile();
            read_frags(As[nxt], Bs[nxt], 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfmas(1);
        __builtin_amdgcn_sched_barrier(0);
    };

    if (nk > 0) {
        load_tile();
        park_tile(As[0], Bs[0]);
        if (nk > 1) load_tile();
        lds_barrier();
        read_frags(As[0], Bs[0], 0);
    }
    int64_t kt = 0;
    for (; kt + 3 < nk; kt += 2) {                                  // every tile the two steps ask for exists
        step(std::integral_constant<int, 0>(), kt, std::true_type());
        step(std::integral_constant<int, 1>(), kt + 1, std::true_type());
    }
    for (; kt < nk; kt += 2) {
        step(std::integral_constant<int, 0>(), kt, std::false_type());
        if (kt + 1 < nk) step(std::integral_constant<int, 1>(), kt + 1, std::false_type());
    }

    float *cbase;
    int64_t ldc;
    if (g.split_k > 1) {
        cbase = partial + ((int64_t)batch * g.split_k + split) * g.rows * g.cols;
        ldc = g.cols;
    } else {
        cbase = g.c + (int64_t)batch * g.stride_c;
        ldc = g.ldc;
    }
    // The MFMAs ran with the operands swapped (B fragment as the 32 x 2 operand), so a tile of the accumulator is
    // the transpose of the output tile: lane l holds output row l % 32 and, in registers 4 g .. 4 g + 3, the four
    // consecutive columns 8 g + 4 (l / 32) + 0..3: one 16-byte store each, a quarter of the store instructions
    // that one register per store would need.
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t row = bm + (BM == 64 ? 0 : wm * 64) + i * 32 + r;
#pragma unroll
        for (int t = 0; t < TN; ++t)
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                const int64_t col = bn + wn * (32 * TN) + t * 32 + 8 * gq + 4 * h;
                floatx4 v;
                v[0] = acc[i][t][4 * gq + 0]; v[1] = acc[i][t][4 * gq + 1];
                v[2] = acc[i][t][4 * gq + 2]; v[3] = acc[i][t][4 * gq + 3];
                *(floatx4 *)(cbase + row * ldc + col) = v;
            }
    }
}

__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float *__restrict__ partial, GemmArgs g, int batch_count)
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

extern "C" int pccnn_gemm_f32(const float *a, const float *b, float *c, int64_t rows, int64_t cols, int64_t inner,
                              int a_trans, int b_trans, int64_t lda, int64_t ldb, int64_t ldc, int batch,
                              int64_t stride_a, int64_t stride_b, int64_t stride_c, int split_k, void *workspace,
                              size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(rows >= 0 && cols >= 0 && inner >= 0 && batch >= 1, PCCNN_ERR_INVALID,
                  "pccnn_gemm_f32: rows=%lld cols=%lld inner=%lld batch=%d", (long long)rows, (long long)cols,
                  (long long)inner, batch);
    if (rows == 0 || cols == 0) return PCCNN_OK;
    PCCNN_REQUIRE(a && b && c, PCCNN_ERR_INVALID, "pccnn_gemm_f32: null pointer");
    PCCNN_REQUIRE(lda >= (a_trans ? rows : inner) && ldb >= (b_trans ? inner : cols) && ldc >= cols, PCCNN_ERR_INVALID,
                  "pccnn_gemm_f32: leading dimension too small (lda=%lld ldb=%lld ldc=%lld)", (long long)lda,
                  (long long)ldb, (long long)ldc);
    if (split_k < 1) split_k = 1;
    GemmArgs g;
    g.a = a; g.b = b; g.c = c;
    g.rows = rows; g.cols = cols; g.inner = inner;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.stride_a = stride_a; g.stride_b = stride_b; g.stride_c = stride_c;
    int64_t chunk = pccnn_ceil_div(pccnn_ceil_div(inner > 0 ? inner : 1, split_k), GT_K) * GT_K;
    split_k = (int)pccnn_ceil_div(inner > 0 ? inner : 1, chunk);
    g.split_k = split_k;
    g.k_chunk = chunk;
    g.aligned = ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0) && (lda % 4 == 0) && (ldb % 4 == 0) &&
                (stride_a % 4 == 0) && (stride_b % 4 == 0);
    // units run along the reduction index where that is contiguous in memory, else along the rows / columns
    g.whole_units = g.aligned && ((a_trans ? rows : inner) % 4 == 0) && ((b_trans ? inner : cols) % 4 == 0);
    float *partial = nullptr;
    if (split_k > 1) {
        size_t need = (size_t)batch * split_k * rows * cols * sizeof(float);
        PCCNN_REQUIRE(workspace && workspace_bytes >= need, PCCNN_ERR_WORKSPACE,
                      "pccnn_gemm_f32: split-k workspace of %zu bytes, need %zu", workspace_bytes, need);
        partial = (float *)workspace;
    }
    hipStream_t s = (hipStream_t)stream;
    // The kernel for full tiles takes every shape that has them, except products with fewer than 12 k tiles per
    // workgroup: there the prologue and the epilogue weigh more than the loop, and the general kernel, which
    // keeps four instead of three waves per SIMD, is ahead (65 536 x 1024 x 128, B transposed: 162 against 166 us).
    // Lane offsets inside a tile are 32-bit byte offsets: 256 rows of the leading dimension must fit.
    const bool full_128 = rows % 128 == 0, full_64 = rows % 64 == 0;
    const bool full_ok = g.aligned && cols % GT_N == 0 && inner % GT_K == 0 && chunk >= 12 * GT_K && lda < (1ll << 20) &&
                         ldb < (1ll << 20) &&
                         (split_k > 1 ? (uintptr_t)partial % 16 == 0
                                      : ldc % 4 == 0 && (uintptr_t)c % 16 == 0 && stride_c % 4 == 0);
    // 128-row tiles unless that leaves the chip short of workgroups: the general kernel wants about four per CU,
    // the kernel for full tiles is ahead with 128-row tiles from one per CU on (65 536 x 128 x 1024: 140 against
    // 153 us with 64-row tiles; the wider tile needs fewer load instructions per MFMA)
    const int64_t wg128 = pccnn_ceil_div(cols, GT_N) * pccnn_ceil_div(rows, 128) * batch * split_k;
    int bm_tile = wg128 >= 1024 ? 128 : 64;
    bool full_tiles = false;
    if (full_ok && full_128 && wg128 >= 256) { bm_tile = 128; full_tiles = true; }
    else if (full_ok && full_64 && bm_tile == 64) full_tiles = true;
    g.tiles_x = (int)pccnn_ceil_div(cols, GT_N);
    g.tiles_y = (int)pccnn_ceil_div(rows, bm_tile);
    g.total_wg = (int64_t)g.tiles_x * g.tiles_y * batch * split_k;
    PCCNN_REQUIRE(g.total_wg < (1ll << 31) - GEMM_XCDS, PCCNN_ERR_UNSUPPORTED, "pccnn_gemm_f32: grid too large");
    dim3 grid((unsigned)(pccnn_ceil_div(g.total_wg, GEMM_XCDS) * GEMM_XCDS));
    {
        PccnnTimed timed(PCCNN_T_GEMM, s);
#define GEMM_GO(AT, BT)                                                                       \
    do {                                                                                      \
        if (full_tiles) {                                                                     \
            if (bm_tile == 128) gemm_f32_full_tiles_kernel<AT, BT, 128><<<grid, 256, 0, s>>>(g, partial); \
            else gemm_f32_full_tiles_kernel<AT, BT, 64><<<grid, 256, 0, s>>>(g, partial);     \
        } else if (bm_tile == 128) gemm_f32_mfma_kernel<AT, BT, 128><<<grid, 256, 0, s>>>(g, partial); \
        else gemm_f32_mfma_kernel<AT, BT, 64><<<grid, 256, 0, s>>>(g, partial);                 \
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
        splitk_reduce_kernel<<<(unsigned)blocks, 256, 0, s>>>(partial, g, batch);
        PCCNN_LAUNCH_CHECK();
    }
    return PCCNN_OK;
}
