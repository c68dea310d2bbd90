// Forward convolution with the projection kept on chip (optional, see pccnn_set_fused_forward): for a tile of 64 samples the gather-aggregate builds one
// 256-column slice of P = [M, Cin*K] in LDS and the matrix cores multiply it with the matching rows of W right
// away, slice after slice, so that P never travels to memory (the reference materialises it:
// pccnn_lib_ops/pcconvs/kpconv.cu:52-57, mcconv.cu:58-68).  Used for forward calls that do not have to hand the
// projection to a backward call; calls that do keep the two-kernel path of conv.hip.
//
//  * Slice = 16 features x 16 basis functions (K <= 16, padded).  A wavefront works on four pairs at a time, one per
//    row of 16 lanes: lane (row, j) evaluates basis function j of its row's pair, loads feature 16 slice + j of the
//    pair's point (the 16 lanes of a row read 64 contiguous bytes) and needs the products of its feature with all 16
//    basis values of the row - which sit in the other 15 lanes of the row: 15 v_fmac_f32 with a DPP row rotation on
//    the basis operand take them from there, so nothing goes through LDS.  Accumulator r of lane j therefore holds
//    basis function (j +- r) mod 16; the rotation is undone by the address the sum is stored to.
//  * A workgroup is 4 wavefronts; each builds 16 of the tile's 64 rows.  Offsets, densities and point ids of its
//    stretch of the pair list are parked in LDS once per tile (up to 192 pairs; longer stretches in batches, once
//    per slice); the feature loads of the next segment of up to 32 pairs are in flight while one is processed.
//  * Contraction: v_mfma_f32_32x32x2_f32 (or v_mfma_f32_32x32x16_bf16 on a bf16 tile).  The A fragments are
//    16-byte LDS reads of the tile (chunk slot XOR row, conflict-free); the B fragments come straight from memory:
//    the weights are first repacked (conv_pack_weights_kernel) so that the four (eight) values a lane feeds to
//    consecutive MFMAs are one 16-byte load, and so that rows for padded basis functions / features read as zeros.
//  * 64 KB (32 KB) of tile + 15 KB of staging: two (three) workgroups per CU, one gathering while another multiplies.
#include <atomic>
#include <type_traits>

#include "conv_basis.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

#define FUSED_TM 64             // samples per workgroup
#define FUSED_CH 256            // columns of P per slice: 16 features x 16 basis functions
#define FUSED_BATCH 192         // pairs staged per wavefront at a time
#define FUSED_SEG 32            // pairs whose feature loads are issued together (8 per lane row)

// Packed weights.  Local column cl of slice s is feature 16 s + cl / 16, basis function cl % 16.
// fp32: [slice][g = 0..31][nt = 0..Cout/32-1][lane][e = 0..3] with lane = (h, c): cl = 8g + 4h + e,
//   value = W[(16 s + cl / 16) * K + cl % 16][32 nt + c];
// bf16: [slice][g = 0..15][nt][lane][e = 0..7], cl = 16g + 8h + e.  Rows outside W (feature >= Cin, basis
// function >= K) are zeros.
template <bool BF16>
__global__ void __launch_bounds__(256)
conv_pack_weights_kernel(const float *__restrict__ w, void *__restrict__ packed, int c_in, int k, int c_out,
                         int64_t total)
{
    constexpr int PER = BF16 ? 8 : 4;                   // values per lane and group
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int nts = c_out / 32;
    const int e = (int)(i % PER);
    const int lane = (int)((i / PER) % 64);
    const int nt = (int)((i / (PER * 64)) % nts);
    const int64_t rest = i / ((int64_t)PER * 64 * nts);
    const int groups = FUSED_CH / (2 * PER);
    const int g = (int)(rest % groups);
    const int slice = (int)(rest / groups);
    const int h = lane >> 5, c = lane & 31;
    const int cl = 2 * PER * g + PER * h + e;
    const int f = 16 * slice + cl / 16, kk = cl % 16;
    float v = 0.0f;
    if (f < c_in && kk < k) v = w[((int64_t)f * k + kk) * c_out + 32 * nt + c];
    if (BF16) ((uint16_t *)packed)[i] = pccnn_bf16_bits(v);
    else ((float *)packed)[i] = v;
}

struct FusedArgs {
    const float *feats;
    const void *packed;     // weights as conv_pack_weights_kernel leaves them
    float *out;             // [m, c_out]
    int c_out;
    int slices;             // ceil(c_in / 16)
    int divide_by_count;    // out rows divided by the sample's pair count
};

// acc[r] += (basis value of the lane r places further round the row of 16) * fv, r = 1..15.  The DPP operand must
// not have been written by the instruction just before (two wait states), hence the s_nop.
#define FUSED_FMAC(r) "v_fmac_f32_dpp %" #r ", %16, %17 row_ror:" #r " row_mask:0xf bank_mask:0xf\n"
__device__ __forceinline__ void fused_row_fmac(float (&acc)[16], float w, float fv)
{
    acc[0] += w * fv;
    asm volatile("s_nop 1\n" FUSED_FMAC(1) FUSED_FMAC(2) FUSED_FMAC(3) FUSED_FMAC(4) FUSED_FMAC(5) FUSED_FMAC(6)
                 FUSED_FMAC(7) FUSED_FMAC(8) FUSED_FMAC(9) FUSED_FMAC(10) FUSED_FMAC(11) FUSED_FMAC(12) FUSED_FMAC(13)
                 FUSED_FMAC(14) FUSED_FMAC(15)
                 : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]),
                   "+v"(acc[7]), "+v"(acc[8]), "+v"(acc[9]), "+v"(acc[10]), "+v"(acc[11]), "+v"(acc[12]),
                   "+v"(acc[13]), "+v"(acc[14]), "+v"(acc[15])
                 : "v"(w), "v"(fv));
}

// WM x WN wavefronts, each TI x TJ MFMA tiles of 32 x 32: 64 = 32 WM TI rows, c_out = 32 WN TJ columns.
template <int BASIS, bool BF16, int WM, int WN, int TI, int TJ>
__global__ void __launch_bounds__(256)
conv_fused_fwd_kernel(ConvGeom g, FusedArgs a)
{
    static_assert(WM * WN == 4 && WM * TI == 2, "four wavefronts cover 64 rows");
    using tile_t = typename std::conditional<BF16, uint16_t, float>::type;
    // tile[m][slot * U + e]: 16-byte unit `q` of row m sits in slot q ^ (m & 15)   (U = 4 floats or 8 bf16)
    __shared__ __attribute__((aligned(16))) tile_t tile[FUSED_TM * FUSED_CH];
    __shared__ __attribute__((aligned(16))) float4 geo_lds[4][FUSED_BATCH];     // (offset, density) per pair
    __shared__ int n_lds[4][FUSED_BATCH];                                       // and its point
    constexpr bool GEOM = BASIS != BASIS_EXPLICIT;
    constexpr int U = BF16 ? 8 : 4;                     // elements per 16-byte unit
    constexpr int UNITS = FUSED_CH / U;                 // units per row: 64 (fp32) or 32 (bf16)

    const int lane = pccnn_lane();
    // (readfirstlane: the wavefront's index and what follows from it are the same in all 64 lanes, which lets the
    // loops below run on scalar registers instead of under per-lane masks)
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int64_t tile_id = pccnn_xcd_block(blockIdx.x, gridDim.x, 8);
    const int64_t s0 = tile_id * FUSED_TM;
    if (s0 >= g.m) return;                              // padding of the launch (uniform for the workgroup)

    // ---- this wavefront's 16 rows and its stretch of the pair list
    const int64_t r0 = s0 + 16 * wave;                  // first sample of the wavefront
    int my_end = 0;                                     // lane l < 16: end of sample r0 + l (clamped to the last sample)
    {
        int64_t s = r0 + (lane & 15);
        if (s > g.m - 1) s = g.m - 1;
        my_end = g.ends[s];
    }
    const int rows_here = (r0 >= g.m) ? 0 : (int)((g.m - r0) < 16 ? (g.m - r0) : 16);
    const int p_begin = __builtin_amdgcn_readfirstlane((r0 > 0 && r0 <= g.m) ? g.ends[(r0 < g.m ? r0 : g.m) - 1] : 0);
    const int p_end = rows_here > 0 ? pccnn_bcast_i(my_end, rows_here - 1) : p_begin;
    float ir0 = 1.f, ir1 = 1.f, ir2 = 1.f;
    if (GEOM) { ir0 = 1.0f / g.radii[0]; ir1 = 1.0f / g.radii[1]; ir2 = 1.0f / g.radii[2]; }

    const int prow = lane >> 4, fl = lane & 15;         // row of 16 lanes = pair slot; place in the row
    LaneBasis<BASIS> lb;
    lb.load(g, fl);                                     // this lane evaluates basis function fl of its row's pair
    // which way row_ror turns: lane fl reads lane fl + dir
    const int dir = (__builtin_amdgcn_update_dpp(0, fl, PCCNN_DPP_ROW_ROR(1), 0xf, 0xf, true) == ((fl + 1) & 15)) ? 1 : -1;

    // offsets, densities and point ids of the pairs b0 .. b1 - 1, one pair per lane
    auto stage = [&](int b0, int b1) {
#pragma unroll
        for (int r = 0; r < FUSED_BATCH / 64; ++r) {
            const int j = 64 * r + lane;
            const int t = b0 + j;
            if (t < b1) {
                const int2 pr = g.neigh[t];
                float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
                if (GEOM) {
                    dx = (g.pts[(int64_t)pr.x * 3 + 0] - g.samples[(int64_t)pr.y * 3 + 0]) * ir0;
                    dy = (g.pts[(int64_t)pr.x * 3 + 1] - g.samples[(int64_t)pr.y * 3 + 1]) * ir1;
                    dz = (g.pts[(int64_t)pr.x * 3 + 2] - g.samples[(int64_t)pr.y * 3 + 2]) * ir2;
                }
                if (BasisTraits<BASIS>::uses_pdf) pd = g.pdf[pr.x];
                geo_lds[wave][j] = make_float4(dx, dy, dz, pd);
                n_lds[wave][j] = pr.x;
            }
        }
        __builtin_amdgcn_wave_barrier();                // (a wavefront's LDS accesses complete in program order)
    };
    const bool single = (p_end - p_begin) <= FUSED_BATCH;       // the common case: staged once for all slices
    if (single) stage(p_begin, p_end);

    const int wm = wave / WN, wn = wave % WN;
    const int h = lane >> 5, c = lane & 31;
    floatx16 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
    const int nts = a.c_out / 32;

    for (int slice = 0; slice < a.slices; ++slice) {
        const int f = 16 * slice + fl;
        const bool fvalid = f < g.c_in;

        // ---------------- gather-aggregate: rows 16 wave .. 16 wave + 15 of the slice
        float pa[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) pa[r] = 0.0f;
        int row = 0;                                    // next row of the wavefront to finish
        // row `r` is complete: add up the four pair slots and store its 256 values
        auto flush = [&](int r) {
            const int m = 16 * wave + r;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // lanes of lane-row prow receive the sum of accumulator 4q + pccnn_rows4_slot(prow)
                const float sum = pccnn_rows4_sum(pa[4 * q], pa[4 * q + 1], pa[4 * q + 2], pa[4 * q + 3]);
                const int kk = (fl + dir * (4 * q + pccnn_rows4_slot(prow))) & 15;
                const int cl = fl * 16 + kk;
                const int at = (m * UNITS + ((cl / U) ^ (m & 15))) * U + (cl % U);
                if (BF16) tile[at] = (tile_t)pccnn_bf16_bits(sum);
                else tile[at] = (tile_t)sum;
            }
#pragma unroll
            for (int q = 0; q < 16; ++q) pa[q] = 0.0f;
        };
        int b0 = p_begin;
        do {
            const int b1 = (p_end - b0) < FUSED_BATCH ? p_end : b0 + FUSED_BATCH;
            if (!single) stage(b0, b1);
            auto row_end = [&](int r) { return pccnn_bcast_i(my_end, r); };
            // next segment at or after `pos`: pairs pos .. e - 1 of row r (at most FUSED_SEG, inside the batch)
            auto next_seg = [&](int pos, int &r, int &e) {
                while (r < rows_here && row_end(r) <= pos) ++r;
                if (r >= rows_here || pos >= b1) return false;
                const int re = row_end(r);
                e = pos + FUSED_SEG;
                if (e > re) e = re;
                if (e > b1) e = b1;
                return true;
            };
            // feature values of a segment: group u holds pair p + 4u + prow
            auto seg_loads = [&](int p, int e, float (&buf)[FUSED_SEG / 4]) {
#pragma unroll
                for (int u = 0; u < FUSED_SEG / 4; ++u) {
                    const int t = p + 4 * u + prow;
                    buf[u] = (fvalid && t < e) ? a.feats[(int64_t)n_lds[wave][t - b0] * g.c_in + f] : 0.0f;
                }
            };
            float cur[FUSED_SEG / 4], nxt[FUSED_SEG / 4];
            int spos = b0, srow = row, send = b0;
            bool have = next_seg(spos, srow, send);
            if (have) seg_loads(spos, send, cur);
            while (have) {
                int nrow = srow, nend = send;
                const bool more = next_seg(send, nrow, nend);
                if (more) seg_loads(send, nend, nxt);
                while (row < srow) { flush(row); ++row; }           // rows without pairs before this one
#pragma unroll
                for (int u = 0; u < FUSED_SEG / 4; ++u) {
                    if (spos + 4 * u < send) {                      // uniform
                        const int t = spos + 4 * u + prow;
                        const bool valid = t < send;
                        float4 ge = make_float4(0.f, 0.f, 0.f, 1.f);
                        if (valid && GEOM) ge = geo_lds[wave][t - b0];
                        const float w = valid ? pair_basis<BASIS>(g, lb, t, ge.x, ge.y, ge.z, ge.w) : 0.0f;
                        fused_row_fmac(pa, w, cur[u]);
                    }
                }
                if (send == row_end(srow)) { flush(row); ++row; }   // that was the row's last segment
                spos = send;
                srow = nrow;
                send = nend;
                have = more;
#pragma unroll
                for (int u = 0; u < FUSED_SEG / 4; ++u) cur[u] = nxt[u];
            }
            // rows without pairs at the end of the batch
            while (row < rows_here && row_end(row) <= b1) { flush(row); ++row; }
            __builtin_amdgcn_wave_barrier();
            b0 = b1;
        } while (b0 < p_end);
        // rows past the last sample (the last tile only): zeros, so that the MFMAs read defined values
        for (int r = rows_here; r < 16; ++r) {
            const int m = 16 * wave + r;
            if (BF16) { if (lane < UNITS) *(uint4 *)&tile[(m * UNITS + lane) * U] = make_uint4(0, 0, 0, 0); }
            else *(float4 *)&tile[(m * UNITS + lane) * U] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
        __syncthreads();

        // ---------------- contraction of the slice: acc += tile[64 x 256] x W[256 rows of the slice]
        if (BF16) {
            constexpr int GROUPS = FUSED_CH / 16;       // one MFMA of 16 k per group
            const uint4 *wp = (const uint4 *)a.packed + ((int64_t)slice * GROUPS * nts + (wn * TJ)) * 64 + lane;
            uint4 bq[2][TJ];
#pragma unroll
            for (int j = 0; j < TJ; ++j) bq[0][j] = wp[(int64_t)j * 64];
#pragma unroll
            for (int gq = 0; gq < GROUPS; ++gq) {
                const int cur = gq & 1;
                if (gq + 1 < GROUPS) {
#pragma unroll
                    for (int j = 0; j < TJ; ++j) bq[cur ^ 1][j] = wp[((int64_t)(gq + 1) * nts + j) * 64];
                }
                uint4 aq[TI];
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const int m = 32 * (wm * TI + i) + c;
                    aq[i] = *(const uint4 *)&tile[(m * UNITS + ((2 * gq + h) ^ (m & 15))) * U];
                }
#pragma unroll
                for (int i = 0; i < TI; ++i)
#pragma unroll
                    for (int j = 0; j < TJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, aq[i]),
                                                                            __builtin_bit_cast(bf16x8, bq[cur][j]),
                                                                            acc[i][j], 0, 0, 0);
            }
        } else {
            constexpr int GROUPS = FUSED_CH / 8;        // four MFMAs of 2 k per group
            const float4 *wp = (const float4 *)a.packed + ((int64_t)slice * GROUPS * nts + (wn * TJ)) * 64 + lane;
            float4 bq[2][TJ];
#pragma unroll
            for (int j = 0; j < TJ; ++j) bq[0][j] = wp[(int64_t)j * 64];
#pragma unroll 4
            for (int gq = 0; gq < GROUPS; ++gq) {
                const int cur = gq & 1;
                if (gq + 1 < GROUPS) {
#pragma unroll
                    for (int j = 0; j < TJ; ++j) bq[cur ^ 1][j] = wp[((int64_t)(gq + 1) * nts + j) * 64];
                }
                float4 aq[TI];
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const int m = 32 * (wm * TI + i) + c;
                    aq[i] = *(const float4 *)&tile[(m * UNITS + ((2 * gq + h) ^ (m & 15))) * U];
                }
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < TI; ++i)
#pragma unroll
                        for (int j = 0; j < TJ; ++j) {
                            const float av = e == 0 ? aq[i].x : (e == 1 ? aq[i].y : (e == 2 ? aq[i].z : aq[i].w));
                            const float bv = e == 0 ? bq[cur][j].x
                                                    : (e == 1 ? bq[cur][j].y : (e == 2 ? bq[cur][j].z : bq[cur][j].w));
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
                        }
            }
        }
        __syncthreads();                                // the tile is free for the next slice
    }

    // ---- results: register v of lane (h, c) holds row 8 (v / 4) + 4 h + v % 4, column c of its 32 x 32 tile
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t s = s0 + 32 * (wm * TI + i) + 8 * (v / 4) + 4 * h + (v % 4);
            if (s < g.m) {
                float scale = 1.0f;
                if (a.divide_by_count) {
                    const int cnt = g.ends[s] - (s > 0 ? g.ends[s - 1] : 0);
                    scale = 1.0f / (float)(cnt > 0 ? cnt : 1);
                }
#pragma unroll
                for (int j = 0; j < TJ; ++j)
                    a.out[s * a.c_out + 32 * (wn * TJ + j) + c] = a.divide_by_count ? acc[i][j][v] * scale : acc[i][j][v];
            }
        }
}

// ------------------------------------------------------------------------------- host side

// Off unless asked for.  Measured on MI355X against the two-kernel path (projection kernel + MFMA GEMM), 65 536
// samples, 0.92 M pairs, 64 -> 128 channels, 16 basis functions: 381 against 237 us in fp32, 278 against 122 us with
// bf16 operands (8 x 8192 points, 1.25 M pairs, 128 -> 256, 15 kernel points: 1158 against 712 us).  The tile and the
// staging take 80 KB of LDS per workgroup, which leaves two wavefronts per SIMD for a gather whose stand-alone
// kernel hides its dependent loads (offsets -> pairs -> positions and feature rows) behind eight; every slice also
// walks the pair list again and pays a cross-row reduction per sample.  What the fusion saves - writing P and
// reading it back, 2 x 268 MB at the first of these shapes - costs the two-kernel path about 50 us.
static std::atomic<int> g_fused_forward{0};

// 1 lets eligible forward calls take the fused kernel, 0 (the default) sends every call down the two-kernel path.
extern "C" int pccnn_set_fused_forward(int on)
{
    return g_fused_forward.exchange(on != 0 ? 1 : 0);
}

bool pccnn_conv_fused_eligible(int basis, int c_in, int k, int num_mlps, int c_out)
{
    if (!g_fused_forward.load(std::memory_order_relaxed) || num_mlps != 1 || basis == BASIS_SPH || basis == BASIS_LINEAR) return false;
    if (k > 16) return false;                           // a slice holds 16 basis functions
    if (c_in < 33) return false;                        // few features: the pair-parallel narrow kernels
    return c_out == 64 || c_out == 128 || c_out == 256;
}

size_t pccnn_conv_fused_workspace_bytes(int c_in, int k, int c_out)
{
    const size_t slices = (size_t)((c_in + 15) / 16);
    (void)k;
    return pccnn_align(slices * FUSED_CH * c_out * sizeof(float));
}

template <int BASIS, bool BF16>
static int fused_launch(const ConvGeom &g, const FusedArgs &a, hipStream_t s)
{
    const int64_t tiles = (g.m + FUSED_TM - 1) / FUSED_TM;
    const unsigned grid = pccnn_xcd_grid(tiles, 8);
    switch (a.c_out) {
    case 64: conv_fused_fwd_kernel<BASIS, BF16, 2, 2, 1, 1><<<grid, 256, 0, s>>>(g, a); break;
    case 128: conv_fused_fwd_kernel<BASIS, BF16, 1, 4, 2, 1><<<grid, 256, 0, s>>>(g, a); break;
    default: conv_fused_fwd_kernel<BASIS, BF16, 1, 4, 2, 2><<<grid, 256, 0, s>>>(g, a); break;
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// out = conv(g, feats, weights) with the projection kept on chip.  The caller has checked
// pccnn_conv_fused_eligible; `workspace` holds pccnn_conv_fused_workspace_bytes bytes for the packed weights.
template <int BASIS>
int pccnn_conv_fused_forward(const ConvGeom &g, const float *feats, const float *weights, int c_out, float *out,
                             void *workspace, bool divide_by_count, bool bf16, hipStream_t s)
{
    if (g.m == 0) return PCCNN_OK;
    FusedArgs a;
    a.feats = feats;
    a.packed = workspace;
    a.out = out;
    a.c_out = c_out;
    a.slices = (g.c_in + 15) / 16;
    a.divide_by_count = divide_by_count ? 1 : 0;
    const int64_t total = (int64_t)a.slices * FUSED_CH * c_out;
    PccnnTimed timed(PCCNN_T_FUSED_FWD, s);
    if (bf16) conv_pack_weights_kernel<true><<<(unsigned)pccnn_ceil_div(total, 256), 256, 0, s>>>(
                  weights, workspace, g.c_in, g.k, c_out, total);
    else conv_pack_weights_kernel<false><<<(unsigned)pccnn_ceil_div(total, 256), 256, 0, s>>>(
             weights, workspace, g.c_in, g.k, c_out, total);
    PCCNN_LAUNCH_CHECK();
    return bf16 ? fused_launch<BASIS, true>(g, a, s) : fused_launch<BASIS, false>(g, a, s);
}

template int pccnn_conv_fused_forward<BASIS_KP>(const ConvGeom &, const float *, const float *, int, float *, void *,
                                                bool, bool, hipStream_t);
template int pccnn_conv_fused_forward<BASIS_MLP>(const ConvGeom &, const float *, const float *, int, float *, void *,
                                                 bool, bool, hipStream_t);
template int pccnn_conv_fused_forward<BASIS_KPN>(const ConvGeom &, const float *, const float *, int, float *, void *,
                                                 bool, bool, hipStream_t);
template int pccnn_conv_fused_forward<BASIS_GAUSS>(const ConvGeom &, const float *, const float *, int, float *, void *,
                                                   bool, bool, hipStream_t);
template int pccnn_conv_fused_forward<BASIS_EXPLICIT>(const ConvGeom &, const float *, const float *, int, float *,
                                                      void *, bool, bool, hipStream_t);
