// KPConv / MCConv: basis projection and neighbor gather-aggregate (forward and backward), plus
// the host entry points that chain them with the fp32 MFMA contraction.
//
// Forward, per sample s:  P[s][f][k] = sum over the pairs t of s of  F[n_t][f] * w[t][k]
//   * one wavefront per (sample, block of 64 input features): lane l owns feature f = 64*fb + l
//     and keeps the K partial sums of its feature in registers;
//   * the pair geometry (neighbor id, normalised offset, density) of up to 64 pairs is loaded
//     lane-parallel; the basis values w[t][0..K) of the chunk are evaluated once, K lanes per pair,
//     and staged in LDS, from where every lane reads them as broadcasts, while the feature row of
//     each neighbor is one coalesced read;
//   * P is stored k-fastest, i.e. row f*K + k of the contraction, then out = P x W on MFMA.
// Backward: dP = dOut x W^T and dW = P^T x dOut on MFMA; a second per-sample walk turns dP into
// feature gradients (coalesced float atomics per neighbor row) and per-pair basis gradients
// (feature rows staged in LDS, K-lane partial sums); a per-sample kernel then applies the basis
// derivative and accumulates point, sample, density and basis-parameter gradients.
#include "common.h"
#include "conv_basis.h"

// Sample lists usually come in a spatial order (pooled points and sorted clouds are in cell order), and neighboring
// samples share most of their neighbors: runs of CONV_XCD_CHUNK consecutive samples go to one XCD (see
// pccnn_xcd_block), whose L2 then holds what they share.  8 x 10^5 points in 8 clouds, 34 123 samples, 8 M pairs,
// 8 features, forward / backward projection: 130 / 379 us with every XCD's workgroups spread over the whole list
// (584 MiB of L2 fetches per forward launch, against 100 MB of pairs and points), 110 / 373 us with runs of 512.
// Eight runs of m / 8 give 103 / 351 us there - one cloud per XCD - but 224 instead of 198 us on 8 x 8192 points in
// no spatial order with 128 features (few pairs, large tiles); runs of 2048 give 116 / 386 us, the short last round
// of runs landing on one XCD; eight runs of equal numbers of pairs, cut by a search in `ends`, 104 / 373 us.
#ifndef CONV_XCD_CHUNK
#define CONV_XCD_CHUNK 512
#endif
__device__ __forceinline__ int64_t conv_sample_of_block(unsigned block, int64_t m)
{
    return pccnn_xcd_block(block, gridDim.x, CONV_XCD_CHUNK);
}
static inline unsigned conv_sample_blocks(int64_t m) { return pccnn_xcd_grid(m, CONV_XCD_CHUNK); }

typedef float floatx4_t __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------------------- forward

template <int BASIS, int KPAD, bool BF16>
__global__ void __launch_bounds__(64)
conv_proj_fwd_kernel(ConvGeom g, const float *__restrict__ feats, void *__restrict__ proj_out)
{
    // One single-wavefront workgroup per (sample, block of 64 features).  The basis values of up to 64 pairs
    // are evaluated once, KPAD lanes per pair, and parked in LDS; every lane then reads them back as
    // broadcasts (four values per read) while it streams the feature rows of the neighbors.
    constexpr int PARTS = 64 / KPAD;
    constexpr int ROWS = 4;
    __shared__ __attribute__((aligned(16))) float w_lds[64][KPAD];
    __shared__ float4 geo_lds[64];                      // (offset, density) of the chunk's pairs
    const int lane = threadIdx.x;
    const int64_t s = conv_sample_of_block(blockIdx.x, g.m);
    if (s >= g.m) return;                               // (the grid is padded to a multiple of the XCD count)
    const int f = blockIdx.y * 64 + lane;
    const bool fvalid = f < g.c_in;
    const int k = lane % KPAD, part = lane / KPAD;
    const int lo = s > 0 ? g.ends[s - 1] : 0;
    const int hi = g.ends[s];
    constexpr bool GEOM = BASIS != BASIS_EXPLICIT;      // explicit basis values need no positions
    float sx = 0.f, sy = 0.f, sz = 0.f, ir0 = 1.f, ir1 = 1.f, ir2 = 1.f;
    if (GEOM) {
        sx = g.samples[s * 3 + 0]; sy = g.samples[s * 3 + 1]; sz = g.samples[s * 3 + 2];
        ir0 = 1.0f / g.radii[0]; ir1 = 1.0f / g.radii[1]; ir2 = 1.0f / g.radii[2];
    }
    LaneBasis<BASIS> lb;
    lb.load(g, k);

    float acc[KPAD];
#pragma unroll
    for (int q = 0; q < KPAD; ++q) acc[q] = 0.0f;

    // Feature rows of the pairs j0 .. j0 + ROWS - 1 of the chunk (zeros past its end).
    auto load_rows = [&](int j0, int cnt, int nidx, float (&row)[ROWS]) {
#pragma unroll
        for (int u = 0; u < ROWS; ++u) {
            const int bn = pccnn_bcast_i(nidx, (j0 + u) < cnt ? (j0 + u) : 0);
            row[u] = (fvalid && (j0 + u) < cnt) ? feats[(int64_t)bn * g.c_in + f] : 0.0f;
        }
    };

    for (int cb = lo; cb < hi; cb += 64) {
        const int cnt = (hi - cb) < 64 ? (hi - cb) : 64;
        int nidx = 0;
        float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
        if (lane < cnt) nidx = g.neigh[cb + lane].x;
        // the first rows leave before the basis is evaluated; from then on one group is always in flight
        float row[ROWS];
        load_rows(0, cnt, nidx, row);
        if (lane < cnt) {
            if (GEOM) {
                dx = (g.pts[(int64_t)nidx * 3 + 0] - sx) * ir0;
                dy = (g.pts[(int64_t)nidx * 3 + 1] - sy) * ir1;
                dz = (g.pts[(int64_t)nidx * 3 + 2] - sz) * ir2;
            }
            if (BasisTraits<BASIS>::uses_pdf) pd = g.pdf[nidx];
        }
        if (GEOM) geo_lds[lane] = make_float4(dx, dy, dz, pd);
        __syncthreads();
        for (int p = 0; p * PARTS < cnt; ++p) {
            const int j = p * PARTS + part;             // < 64: PARTS divides 64 and p * PARTS < cnt <= 64
            float4 ge = make_float4(0.f, 0.f, 0.f, 1.f);
            if (GEOM) ge = geo_lds[j];
            const float w = (j < cnt) ? pair_basis<BASIS>(g, lb, (int64_t)cb + j, ge.x, ge.y, ge.z, ge.w) : 0.0f;
            w_lds[j][k] = w;
        }
        __syncthreads();
        for (int j0 = 0; j0 < cnt; j0 += ROWS) {
            float row_next[ROWS];
            const bool more = j0 + ROWS < cnt;                      // uniform
            if (more) load_rows(j0 + ROWS, cnt, nidx, row_next);
#pragma unroll
            for (int u = 0; u < ROWS; ++u) {
                if (j0 + u < cnt) {                                 // uniform
#pragma unroll
                    for (int q = 0; q < KPAD; q += 4) {
                        const float4 wv = *(const float4 *)&w_lds[j0 + u][q];
                        acc[q] += row[u] * wv.x;
                        acc[q + 1] += row[u] * wv.y;
                        acc[q + 2] += row[u] * wv.z;
                        acc[q + 3] += row[u] * wv.w;
                    }
                }
            }
            if (more) {
#pragma unroll
                for (int u = 0; u < ROWS; ++u) row[u] = row_next[u];
            }
        }
        __syncthreads();
    }
    // The tile of this workgroup, [features][k], is contiguous in memory: hand the accumulators over through
    // LDS so that every store instruction writes one contiguous run instead of 64 rows' worth of pieces.
    float *tile = &w_lds[0][0];
#pragma unroll
    for (int q = 0; q < KPAD; q += 4)
        *(float4 *)&tile[lane * KPAD + q] = make_float4(acc[q], acc[q + 1], acc[q + 2], acc[q + 3]);
    __syncthreads();
    const int f0 = blockIdx.y * 64;
    const int nf = (g.c_in - f0) < 64 ? (g.c_in - f0) : 64;
    const int64_t dst_at = ((int64_t)s * g.c_in + f0) * g.k;
    if (BF16) {
        // the projection leaves as bf16 (round to nearest even): the operand format of the bf16 contraction
        uint16_t *dst = (uint16_t *)proj_out + dst_at;
        if (g.k == KPAD) {
            for (int i = lane; i < nf * (KPAD / 4); i += 64) {
                const float4 v = ((const float4 *)tile)[i];
                uint2 o;
                o.x = pccnn_bf16_bits(v.x) | ((uint32_t)pccnn_bf16_bits(v.y) << 16);
                o.y = pccnn_bf16_bits(v.z) | ((uint32_t)pccnn_bf16_bits(v.w) << 16);
                ((uint2 *)dst)[i] = o;
            }
        } else {
            for (int idx = lane; idx < nf * g.k; idx += 64) {
                const int ff = idx / g.k, q = idx - ff * g.k;
                dst[idx] = pccnn_bf16_bits(tile[ff * KPAD + q]);
            }
        }
    } else {
        float *dst = (float *)proj_out + dst_at;
        if (g.k == KPAD) {
            // whole lines that nothing reads before the next kernel: stored past the L2 (65 536 samples x 64 features
            // x 16: 85 -> 80 us, the contraction behind it 2 us slower).
            // Not for the bf16 tile: half the size, much of it is still in cache when the contraction reads it
            // (40 -> 49 us with such stores).
            for (int i = lane; i < nf * (KPAD / 4); i += 64) {
                const floatx4_t v = ((const floatx4_t *)tile)[i];
                __builtin_nontemporal_store(v, &((floatx4_t *)dst)[i]);
            }
        } else {
            for (int idx = lane; idx < nf * g.k; idx += 64) {
                const int ff = idx / g.k, q = idx - ff * g.k;
                dst[idx] = tile[ff * KPAD + q];
            }
        }
    }
}

// Forward projection for at most 32 input features.  With lane = feature, most of a wavefront would idle; here
// G = 64 / FPAD pairs are processed side by side, lane = (pair slot, feature): every lane keeps K partial sums for
// its feature over the pairs that fall into its slot, and the slots are added at the end (DPP rotations and row
// swaps).  Basis values and pair records go through LDS as in the wide kernel.
template <int BASIS, int KPAD, int FPAD, bool BF16>
__global__ void __launch_bounds__(64)
conv_proj_fwd_narrow_kernel(ConvGeom g, const float *__restrict__ feats, void *__restrict__ proj_out)
{
    constexpr int PARTS = 64 / KPAD;
    constexpr int G = 64 / FPAD;                        // pairs per step
    constexpr int STEPS = 4;                            // steps whose feature loads are in flight together
    __shared__ __attribute__((aligned(16))) float w_lds[64][KPAD];
    __shared__ float4 geo_lds[64];                      // (offset, density) of the chunk's pairs
    __shared__ int nidx_lds[64];                        // and their points
    const int lane = threadIdx.x;
    const int64_t s = conv_sample_of_block(blockIdx.x, g.m);
    if (s >= g.m) return;                               // (the grid is padded to a multiple of the XCD count)
    const int f = lane % FPAD, slot = lane / FPAD;
    const bool fvalid = f < g.c_in;
    const int k = lane % KPAD, part = lane / KPAD;
    const int lo = s > 0 ? g.ends[s - 1] : 0;
    const int hi = g.ends[s];
    constexpr bool GEOM = BASIS != BASIS_EXPLICIT;
    float sx = 0.f, sy = 0.f, sz = 0.f, ir0 = 1.f, ir1 = 1.f, ir2 = 1.f;
    if (GEOM) {
        sx = g.samples[s * 3 + 0]; sy = g.samples[s * 3 + 1]; sz = g.samples[s * 3 + 2];
        ir0 = 1.0f / g.radii[0]; ir1 = 1.0f / g.radii[1]; ir2 = 1.0f / g.radii[2];
    }
    LaneBasis<BASIS> lb;
    lb.load(g, k);
    float acc[KPAD];
#pragma unroll
    for (int q = 0; q < KPAD; ++q) acc[q] = 0.0f;

    for (int cb = lo; cb < hi; cb += 64) {
        const int cnt = (hi - cb) < 64 ? (hi - cb) : 64;
        int nidx = 0;
        float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
        if (lane < cnt) {
            nidx = g.neigh[cb + lane].x;
            if (GEOM) {
                dx = (g.pts[(int64_t)nidx * 3 + 0] - sx) * ir0;
                dy = (g.pts[(int64_t)nidx * 3 + 1] - sy) * ir1;
                dz = (g.pts[(int64_t)nidx * 3 + 2] - sz) * ir2;
            }
            if (BasisTraits<BASIS>::uses_pdf) pd = g.pdf[nidx];
        }
        nidx_lds[lane] = nidx;
        if (GEOM) geo_lds[lane] = make_float4(dx, dy, dz, pd);
        __syncthreads();
        for (int p = 0; p * PARTS < cnt; ++p) {
            const int j = p * PARTS + part;             // < 64: PARTS divides 64 and p * PARTS < cnt <= 64
            float4 ge = make_float4(0.f, 0.f, 0.f, 1.f);
            if (GEOM) ge = geo_lds[j];
            const float w = (j < cnt) ? pair_basis<BASIS>(g, lb, (int64_t)cb + j, ge.x, ge.y, ge.z, ge.w) : 0.0f;
            w_lds[j][k] = w;
        }
        __syncthreads();
        for (int j0 = 0; j0 < cnt; j0 += G * STEPS) {
            float row[STEPS];
#pragma unroll
            for (int u = 0; u < STEPS; ++u) {
                const int j = j0 + u * G + slot;        // < 64 whenever it is below cnt
                row[u] = (fvalid && j < cnt) ? feats[(int64_t)nidx_lds[j & 63] * g.c_in + f] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < STEPS; ++u) {
                const int j = j0 + u * G + slot;
                if (j < cnt) {
#pragma unroll
                    for (int q = 0; q < KPAD; q += 4) {
                        const float4 wv = *(const float4 *)&w_lds[j][q];
                        acc[q] += row[u] * wv.x;
                        acc[q + 1] += row[u] * wv.y;
                        acc[q + 2] += row[u] * wv.z;
                        acc[q + 3] += row[u] * wv.w;
                    }
                }
            }
        }
        __syncthreads();
    }
    // the slots' partial sums, then the tile [features][k] through LDS so that the stores are contiguous runs
#pragma unroll
    for (int q = 0; q < KPAD; ++q) acc[q] = pccnn_strided_sum<FPAD>(acc[q]);
    float *tile = &w_lds[0][0];
    if (slot == 0) {
#pragma unroll
        for (int q = 0; q < KPAD; q += 4)
            *(float4 *)&tile[f * KPAD + q] = make_float4(acc[q], acc[q + 1], acc[q + 2], acc[q + 3]);
    }
    __syncthreads();
    const int nf = g.c_in;
    const int64_t dst_at = (int64_t)s * g.c_in * g.k;
    if (BF16) {
        uint16_t *dst = (uint16_t *)proj_out + dst_at;
        for (int idx = lane; idx < nf * g.k; idx += 64) {
            const int ff = idx / g.k, q = idx - ff * g.k;
            dst[idx] = pccnn_bf16_bits(tile[ff * KPAD + q]);
        }
    } else {
        float *dst = (float *)proj_out + dst_at;
        for (int idx = lane; idx < nf * g.k; idx += 64) {
            const int ff = idx / g.k, q = idx - ff * g.k;
            dst[idx] = tile[ff * KPAD + q];
        }
    }
}

// Derivative of one basis value w.r.t. the pair's normalised offset, the neighbor's density and the basis
// parameters of this lane's k.  gk = upstream gradient of the basis value; (gx, gy, gz, gpdf) receive the
// offset / density gradients, (p0..p3) accumulate the parameter gradients.
template <int BASIS>
__device__ __forceinline__ void basis_derivative(const ConvGeom &g, const LaneBasis<BASIS> &lb, float dx, float dy,
                                                 float dz, float pdf, float gk, float &gx, float &gy, float &gz,
                                                 float &gpdf, float &p0, float &p1, float &p2, float &p3)
{
    // The KPConv correlation has a kink where a pair sits exactly one sigma away from a kernel
    // point, and every self pair (offset 0) does so for the kernel points closest to the centre.
    // Which side of the kink such a pair falls on is decided by the last bit of the fp32
    // distance, so the distance is evaluated exactly as written: no fused multiply-add.
#pragma clang fp contract(off)
    const float c0 = lb.c0, c1 = lb.c1, c2 = lb.c2, c3 = lb.c3;
    if (BASIS == BASIS_KP || BASIS == BASIS_KPN) {
        // kernel_pts_basis_grads; KPConvN feeds it the gradient already divided by the density
        const float gin = (BASIS == BASIS_KPN) ? gk / pdf : gk;
        const float vx = c0 - dx, vy = c1 - dy, vz = c2 - dz;
        const float dist = sqrtf(fmaxf(vx * vx + vy * vy + vz * vz, 0.0f));
        const float res = 1.0f - dist / g.sigma;
        if (res >= 0.0f) {
            const float c = -(gin / g.sigma) * (1.0f / (dist + 1e-6f));
            const float cx = c * vx, cy = c * vy, cz = c * vz;
            gx = -cx; gy = -cy; gz = -cz;
            p0 += cx; p1 += cy; p2 += cz;
        }
    } else if (BASIS == BASIS_GAUSS) {
        const float vx = c0 - dx, vy = c1 - dy, vz = c2 - dz;
        const float e = expf(-((vx * vx + vy * vy + vz * vz) / (2.0f * g.sigma * g.sigma)));
        const float gin = gk / pdf;
        gpdf = -((e / pdf) * gk) / pdf;
        const float c = -gin * e * (1.0f / (g.sigma * g.sigma));
        const float cx = c * vx, cy = c * vy, cz = c * vz;
        gx = -cx; gy = -cy; gz = -cz;
        p0 += cx; p1 += cy; p2 += cz;
    } else if (BASIS == BASIS_MLP) {
        const float inv_pd = 1.0f / pdf;
        float act = dx * c0 + dy * c1 + dz * c2 + c3;
        const bool pos = act > 0.0f;
        act = pos ? act : act * 0.2f;
        gpdf = -(act * gk * inv_pd * inv_pd);
        const float c = gk * inv_pd * (pos ? 1.0f : 0.2f);
        gx = c * c0; gy = c * c1; gz = c * c2;
        p0 += dx * c; p1 += dy * c; p2 += dz * c; p3 += c;
    }
}

// ------------------------------------------------------------------------------ backward

// Backward of the gather-aggregate for one sample per single-wavefront workgroup.
//   dF[n_t][f]  += sum_k dP[s][f][k] * w[t][k]        (lane = feature f, dP row in registers)
//   dw[t][k]     = sum_f dP[s][f][k] * F[n_t][f]      (lane = (k, group of KPAD features), dP column in registers)
// The basis values of up to 32 pairs are evaluated once (KPAD lanes per pair) and parked in LDS, from where
// the dF stage reads them as broadcasts; the neighbor's feature row is read coalesced from memory (the rows of
// the next four pairs travel while four are processed) and handed to the dw stage through LDS, so that each
// stage runs KPAD multiply-adds per pair and lane.  The feature groups' partial sums of dw are added across the
// lanes (row swaps for KPAD = 16) and accumulated in LDS over the feature blocks.
//
// For a basis given by the caller (EXPLICIT) dw is the result and is stored coalesced.  For the parametric
// bases the kernel goes on while the chunk is still in LDS: KPAD lanes per pair apply the basis derivative
// (lane = basis index k), DPP sums over k give the pair's offset / density gradients, and the chunk's values
// are scattered with float atomics, sixteen pairs x (x, y, z, density) per instruction - or, when the caller
// has the mirror index of a symmetric neighborhood, stored per pair for a gather without atomics.  The sample's
// own gradient and the basis-parameter gradients stay in registers until the end; the latter are added to one
// of PARAM_ROWS partial rows ([component][k], 256 floats) that the conv_param_reduce kernels sum afterwards.
#define PARAM_ROWS 256

template <int BASIS, int KPAD, bool want_df, bool want_db>
__global__ void __launch_bounds__(64)
conv_proj_bwd_kernel(ConvGeom g, const float *__restrict__ feats, const float *__restrict__ proj_grads,
                     float *__restrict__ feat_grads, float *__restrict__ basis_grads, float *__restrict__ d_pts,
                     float *__restrict__ d_samples, float *__restrict__ d_pdf, float *__restrict__ param_partials,
                     float *__restrict__ pair_grads)
{
    constexpr bool FUSED = want_db && BasisTraits<BASIS>::differentiable;   // basis derivative applied here
    constexpr int CH = 32;                                          // pairs staged in LDS at a time
    __shared__ __attribute__((aligned(16))) float g_lds[FUSED ? CH : 1][4];
    __shared__ float4 geo_lds[CH];                                  // (offset, density) of the chunk's pairs
    __shared__ int nidx_lds[CH];                                    // and their points
    // want_df / want_db: which of the two stages this instantiation runs
    constexpr int PARTS = 64 / KPAD;                                // feature groups of the dw stage
    constexpr int ROWS = 4;                                         // feature rows in flight
    __shared__ __attribute__((aligned(16))) float w_lds[CH][KPAD];
    __shared__ __attribute__((aligned(16))) float db_lds[want_db ? CH : 1][KPAD];
    __shared__ __attribute__((aligned(16))) float row_lds[want_db ? ROWS : 1][64];
    const int lane = threadIdx.x;
    const int64_t s = conv_sample_of_block(blockIdx.x, g.m);
    if (s >= g.m) return;                               // (the grid is padded to a multiple of the XCD count)
    const int k = lane % KPAD, part = lane / KPAD;
    const int lo = s > 0 ? g.ends[s - 1] : 0;
    const int hi = g.ends[s];
    constexpr bool GEOM = BASIS != BASIS_EXPLICIT;      // explicit basis values need no positions
    float sx = 0.f, sy = 0.f, sz = 0.f, ir0 = 1.f, ir1 = 1.f, ir2 = 1.f;
    if (GEOM) {
        sx = g.samples[s * 3 + 0]; sy = g.samples[s * 3 + 1]; sz = g.samples[s * 3 + 2];
        ir0 = 1.0f / g.radii[0]; ir1 = 1.0f / g.radii[1]; ir2 = 1.0f / g.radii[2];
    }
    LaneBasis<BASIS> lb;
    lb.load(g, k);
    const int fblocks = (g.c_in + 63) / 64;
    // gradients towards positions or densities wanted (uniform): otherwise the per-pair sums over the basis index
    // and their hand-over through LDS are skipped
    const bool geometry = d_pts != nullptr || d_samples != nullptr || d_pdf != nullptr || pair_grads != nullptr;
    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;       // parameter gradients of this lane's k (FUSED)
    float sg = 0.f;                                     // component (lane & 3) of the sample's gradient, unsigned

    // The sample's tile of the projection gradient: row f = this lane's feature (gp, for the dF stage) and column
    // k of the features of this lane's group (gt, for the dw stage).  With one feature block it is loaded once,
    // first thing, so that it travels while the pair list is read.
    auto load_tile = [&](int fb, float (&gp)[KPAD], float (&gt)[KPAD]) {
        const int f = fb * 64 + lane;
#pragma unroll
        for (int q = 0; q < KPAD; ++q) { gp[q] = 0.0f; gt[q] = 0.0f; }
        if (f < g.c_in) {
            const float *src = proj_grads + ((int64_t)s * g.c_in + f) * g.k;
            if (g.k == KPAD && (KPAD % 4) == 0) {
#pragma unroll
                for (int q = 0; q < KPAD; q += 4) {
                    const float4 v = *(const float4 *)(src + q);
                    gp[q] = v.x; gp[q + 1] = v.y; gp[q + 2] = v.z; gp[q + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int q = 0; q < KPAD; ++q)
                    if (q < g.k) gp[q] = src[q];
            }
        }
        if (want_db) {
            if (g.k == KPAD && (g.c_in & 63) == 0) {
                // full tile: one base address, the KPAD loads differ by constants
                const float *col = proj_grads + ((int64_t)s * g.c_in + fb * 64 + part * KPAD) * KPAD + k;
#pragma unroll
                for (int q = 0; q < KPAD; ++q) gt[q] = col[q * KPAD];
            } else if (k < g.k) {
#pragma unroll
                for (int q = 0; q < KPAD; ++q) {
                    const int ft = fb * 64 + part * KPAD + q;
                    if (ft < g.c_in) gt[q] = proj_grads[((int64_t)s * g.c_in + ft) * g.k + k];
                }
            }
        }
    };
    // Feature rows of the pairs j0 .. j0 + ROWS - 1 of the chunk (zeros past its end).
    auto load_rows = [&](int fb, int j0, int cnt, int nidx, float (&row)[ROWS], int (&bn)[ROWS]) {
        const int f = fb * 64 + lane;
#pragma unroll
        for (int u = 0; u < ROWS; ++u) {
            bn[u] = pccnn_bcast_i(nidx, (j0 + u) < cnt ? (j0 + u) : 0);
            row[u] = (f < g.c_in && (j0 + u) < cnt) ? feats[(int64_t)bn[u] * g.c_in + f] : 0.0f;
        }
    };
    float gp[KPAD], gt[KPAD];
    if (hi > lo) load_tile(0, gp, gt);

    for (int cb = lo; cb < hi; cb += CH) {
        const int cnt = (hi - cb) < CH ? (hi - cb) : CH;
        int nidx = 0;
        float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
        if (lane < cnt) nidx = g.neigh[cb + lane].x;
        // the first rows leave before the basis is evaluated; from then on one group is always in flight
        float row[ROWS];
        int bn[ROWS];
        load_rows(0, 0, cnt, nidx, row, bn);
        if (lane < cnt) {
            if (GEOM) {
                dx = (g.pts[(int64_t)nidx * 3 + 0] - sx) * ir0;
                dy = (g.pts[(int64_t)nidx * 3 + 1] - sy) * ir1;
                dz = (g.pts[(int64_t)nidx * 3 + 2] - sz) * ir2;
            }
            if (BasisTraits<BASIS>::uses_pdf) pd = g.pdf[nidx];
        }
        if (lane < CH) {
            if (GEOM) geo_lds[lane] = make_float4(dx, dy, dz, pd);
            nidx_lds[lane] = nidx;
        }
        __syncthreads();
        // basis values of the chunk: pass p evaluates pairs p*PARTS .. p*PARTS + PARTS - 1 (all below CH: PARTS
        // divides CH and p * PARTS < cnt <= CH)
        for (int p = 0; p * PARTS < cnt; ++p) {
            const int j = p * PARTS + part;
            float4 ge = make_float4(0.f, 0.f, 0.f, 1.f);
            if (GEOM) ge = geo_lds[j];
            const float w = (j < cnt) ? pair_basis<BASIS>(g, lb, (int64_t)cb + j, ge.x, ge.y, ge.z, ge.w) : 0.0f;
            w_lds[j][k] = w;
        }
        __syncthreads();
        for (int fb = 0; fb < fblocks; ++fb) {
            const int f = fb * 64 + lane;
            const bool fvalid = f < g.c_in;
            if (fblocks > 1) {
                load_tile(fb, gp, gt);
                if (fb > 0) load_rows(fb, 0, cnt, nidx, row, bn);
            }
            for (int j0 = 0; j0 < cnt; j0 += ROWS) {
                float row_next[ROWS];
                int bn_next[ROWS];
                const bool more = j0 + ROWS < cnt;                  // uniform
                if (more) load_rows(fb, j0 + ROWS, cnt, nidx, row_next, bn_next);
                if (want_db) {
#pragma unroll
                    for (int u = 0; u < ROWS; ++u) row_lds[u][lane] = row[u];
                    __syncthreads();
                }
                if (want_df) {
#pragma unroll
                    for (int u = 0; u < ROWS; ++u) {
                        const int j = j0 + u;
                        if (j < cnt) {                              // uniform
                            float gf = 0.0f;
#pragma unroll
                            for (int q = 0; q < KPAD; q += 4) {
                                const float4 wv = *(const float4 *)&w_lds[j][q];
                                gf += gp[q] * wv.x + gp[q + 1] * wv.y + gp[q + 2] * wv.z + gp[q + 3] * wv.w;
                            }
                            if (fvalid) {
                                if (g.deterministic) __builtin_nontemporal_store(gf, &feat_grads[(int64_t)(cb + j) * g.c_in + f]);
                                else unsafeAtomicAdd(&feat_grads[(int64_t)bn[u] * g.c_in + f], gf);
                            }
                        }
                    }
                }
                if (want_db) {
                    // this lane's share (its KPAD features) of db[j0 + u][k]; rows past the chunk hold zeros
                    float part_sum[ROWS];
#pragma unroll
                    for (int u = 0; u < ROWS; ++u) {
                        float acc = 0.0f;
                        if (j0 + u < cnt) {                         // uniform
#pragma unroll
                            for (int q = 0; q < KPAD; q += 4) {
                                const float4 rv = *(const float4 *)&row_lds[u][part * KPAD + q];
                                acc += gt[q] * rv.x + gt[q + 1] * rv.y + gt[q + 2] * rv.z + gt[q + 3] * rv.w;
                            }
                        }
                        part_sum[u] = acc;
                    }
                    // summed over the feature groups (lanes k, k + KPAD, ...); the first feature block writes
                    if (PARTS == 4 && ROWS == 4) {
                        const float tot = pccnn_rows4_sum(part_sum[0], part_sum[1], part_sum[2], part_sum[3]);
                        const int j = j0 + pccnn_rows4_slot(part);
                        if (j < cnt) db_lds[j][k] = (fb == 0) ? tot : db_lds[j][k] + tot;
                    } else {
#pragma unroll
                        for (int u = 0; u < ROWS; ++u) {
                            const float tot = pccnn_strided_sum<KPAD>(part_sum[u]);
                            if (part == 0 && j0 + u < cnt) db_lds[j0 + u][k] = (fb == 0) ? tot : db_lds[j0 + u][k] + tot;
                        }
                    }
                }
                if (want_db) __syncthreads();
                if (more) {
#pragma unroll
                    for (int u = 0; u < ROWS; ++u) { row[u] = row_next[u]; bn[u] = bn_next[u]; }
                }
            }
        }
        __syncthreads();
        if (FUSED) {
            for (int p = 0; p * PARTS < cnt; ++p) {
                const int j = p * PARTS + part;
                const float4 ge = geo_lds[j];
                float gx = 0.f, gy = 0.f, gz = 0.f, gpdf = 0.f;
                if (j < cnt && lb.active)
                    basis_derivative<BASIS>(g, lb, ge.x, ge.y, ge.z, ge.w, db_lds[j][k], gx, gy, gz, gpdf, p0, p1, p2, p3);
                if (!geometry) continue;                // only the parameters' gradients are asked for
                // summed over the basis index: the KPAD lanes of this pair
                gx = pccnn_group_sum<KPAD>(gx);
                gy = pccnn_group_sum<KPAD>(gy);
                gz = pccnn_group_sum<KPAD>(gz);
                if (BasisTraits<BASIS>::pdf_grad) gpdf = pccnn_group_sum<KPAD>(gpdf);
                if (k < 4) g_lds[j][k] = (k == 0) ? gx * ir0 : (k == 1) ? gy * ir1 : (k == 2) ? gz * ir2 : gpdf;
            }
            __syncthreads();
            for (int i = 0; geometry && i * 16 < cnt; ++i) {
                const int j = i * 16 + (lane >> 2), comp = lane & 3;
                if (j < cnt) {
                    const int jn = nidx_lds[j];
                    const float v = g_lds[j][comp];
                    if (comp < 3) sg += v;
                    if (pair_grads) {
                        // per-pair values, summed per point afterwards by conv_point_gather_kernel
                        pair_grads[(int64_t)(cb + j) * 4 + comp] = v;
                    } else if (comp < 3) {
                        if (d_pts) unsafeAtomicAdd(&d_pts[(int64_t)jn * 3 + comp], v);
                    } else if (BasisTraits<BASIS>::pdf_grad && d_pdf) {
                        unsafeAtomicAdd(&d_pdf[jn], v);
                    }
                }
            }
        } else if (want_db) {
            for (int idx = lane; idx < cnt * KPAD; idx += 64) {
                const int j = idx / KPAD, kk = idx % KPAD;
                if (kk < g.k) basis_grads[(int64_t)(cb + j) * g.k + kk] = db_lds[j][kk];
            }
        }
        __syncthreads();
    }
    if (FUSED) {
        sg = pccnn_strided_sum<4>(sg);
        if (lane < 3 && d_samples) d_samples[s * 3 + lane] = -sg;
        if (param_partials) {
            p0 = pccnn_strided_sum<KPAD>(p0);
            p1 = pccnn_strided_sum<KPAD>(p1);
            p2 = pccnn_strided_sum<KPAD>(p2);
            if (BasisTraits<BASIS>::axis) p3 = pccnn_strided_sum<KPAD>(p3);
            constexpr int COMPS = BasisTraits<BASIS>::axis ? 4 : 3;
            if (g.deterministic) {
                // a compact row [component][KPAD] per sample, summed in a fixed order afterwards
                float *row = param_partials + s * (4 * KPAD);
                for (int c = part; c < 4; c += PARTS)
                    row[c * KPAD + k] = (c == 0) ? p0 : (c == 1) ? p1 : (c == 2) ? p2 : (COMPS == 4 ? p3 : 0.0f);
            } else {
                float *row = param_partials + (int64_t)(blockIdx.x % PARAM_ROWS) * 256;
                for (int c = part; c < COMPS; c += PARTS) {
                    const float v = (c == 0) ? p0 : (c == 1) ? p1 : (c == 2) ? p2 : p3;
                    unsafeAtomicAdd(&row[c * 64 + k], v);
                }
            }
        }
    }
}

// Backward projection for at most 32 input features (arguments and results as conv_proj_bwd_kernel).  Two lane
// layouts, each using the whole wavefront: for dF, lane = (pair slot, feature f) with the f-th row of the sample's
// gradient tile in registers, 64 / FPAD pairs per step; for dw, lane = (pair slot, basis index k) with column k of
// the tile in registers and the pairs' feature rows in LDS, 64 / KPAD pairs per step - the sum over the features
// runs inside the lane, so nothing is added across lanes.
template <int BASIS, int KPAD, int FPAD, bool want_df, bool want_db>
__global__ void __launch_bounds__(64)
conv_proj_bwd_narrow_kernel(ConvGeom g, const float *__restrict__ feats, const float *__restrict__ proj_grads,
                            float *__restrict__ feat_grads, float *__restrict__ basis_grads,
                            float *__restrict__ d_pts, float *__restrict__ d_samples, float *__restrict__ d_pdf,
                            float *__restrict__ param_partials, float *__restrict__ pair_grads)
{
    constexpr bool FUSED = want_db && BasisTraits<BASIS>::differentiable;   // basis derivative applied here
    // pairs staged in LDS at a time: with the feature gradients' atomics in the chunk, 64 (8 x 10^5 points, 8 M pairs,
    // 8 features: 400 -> 377 us); without them 32, where 64 costs occupancy and gains nothing (221 -> 257 us)
    constexpr int CH = want_df ? 64 : 32;
    constexpr int PARTS = 64 / KPAD;                                // pairs per step of the dw / derivative stages
    constexpr int GF = 64 / FPAD;                                   // pairs per step of the dF stage
    constexpr bool GEOM = BASIS != BASIS_EXPLICIT;
    __shared__ __attribute__((aligned(16))) float g_lds[FUSED ? CH : 1][4];
    __shared__ float4 geo_lds[CH];                                  // (offset, density) of the chunk's pairs
    __shared__ int nidx_lds[CH];                                    // and their points
    __shared__ __attribute__((aligned(16))) float w_lds[CH][KPAD];
    __shared__ __attribute__((aligned(16))) float db_lds[want_db ? CH : 1][KPAD];
    __shared__ __attribute__((aligned(16))) float row_lds[want_db ? CH : 1][FPAD];
    const int lane = threadIdx.x;
    const int64_t s = conv_sample_of_block(blockIdx.x, g.m);
    if (s >= g.m) return;                               // (the grid is padded to a multiple of the XCD count)
    const int k = lane % KPAD, part = lane / KPAD;
    const int f = lane % FPAD, slot = lane / FPAD;
    const bool fvalid = f < g.c_in;
    const int lo = s > 0 ? g.ends[s - 1] : 0;
    const int hi = g.ends[s];
    float sx = 0.f, sy = 0.f, sz = 0.f, ir0 = 1.f, ir1 = 1.f, ir2 = 1.f;
    if (GEOM) {
        sx = g.samples[s * 3 + 0]; sy = g.samples[s * 3 + 1]; sz = g.samples[s * 3 + 2];
        ir0 = 1.0f / g.radii[0]; ir1 = 1.0f / g.radii[1]; ir2 = 1.0f / g.radii[2];
    }
    LaneBasis<BASIS> lb;
    lb.load(g, k);
    // gradients towards positions or densities wanted (uniform): otherwise the per-pair sums over the basis index
    // and their hand-over through LDS are skipped
    const bool geometry = d_pts != nullptr || d_samples != nullptr || d_pdf != nullptr || pair_grads != nullptr;
    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;       // parameter gradients of this lane's k (FUSED)
    float sg = 0.f;                                     // component (lane & 3) of the sample's gradient, unsigned
    // the sample's gradient tile: row f (dF stage) and column k (dw stage)
    float gp[KPAD], gt[FPAD];
#pragma unroll
    for (int q = 0; q < KPAD; ++q) gp[q] = 0.0f;
#pragma unroll
    for (int q = 0; q < FPAD; ++q) gt[q] = 0.0f;
    if (hi > lo) {
        const float *tile = proj_grads + (int64_t)s * g.c_in * g.k;
        if (want_df && fvalid) {
#pragma unroll
            for (int q = 0; q < KPAD; ++q)
                if (q < g.k) gp[q] = tile[f * g.k + q];
        }
        if (want_db && k < g.k) {
#pragma unroll
            for (int q = 0; q < FPAD; ++q)
                if (q < g.c_in) gt[q] = tile[q * g.k + k];
        }
    }

    for (int cb = lo; cb < hi; cb += CH) {
        const int cnt = (hi - cb) < CH ? (hi - cb) : CH;
        int nidx = 0;
        float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
        if (lane < cnt) {
            nidx = g.neigh[cb + lane].x;
            if (GEOM) {
                dx = (g.pts[(int64_t)nidx * 3 + 0] - sx) * ir0;
                dy = (g.pts[(int64_t)nidx * 3 + 1] - sy) * ir1;
                dz = (g.pts[(int64_t)nidx * 3 + 2] - sz) * ir2;
            }
            if (BasisTraits<BASIS>::uses_pdf) pd = g.pdf[nidx];
        }
        if (lane < CH) {
            if (GEOM) geo_lds[lane] = make_float4(dx, dy, dz, pd);
            nidx_lds[lane] = nidx;
        }
        __syncthreads();
        if (want_db) {
            // the pairs' feature rows, GF pairs per load instruction (zeros past the last feature)
            for (int j0 = 0; j0 < cnt; j0 += GF) {
                const int j = j0 + slot;
                if (j < cnt) row_lds[j][f] = fvalid ? feats[(int64_t)nidx_lds[j] * g.c_in + f] : 0.0f;
            }
        }
        // basis values of the chunk: pass p evaluates pairs p*PARTS .. p*PARTS + PARTS - 1
        for (int p = 0; p * PARTS < cnt; ++p) {
            const int j = p * PARTS + part;             // < CH: PARTS divides CH and p * PARTS < cnt <= CH
            float4 ge = make_float4(0.f, 0.f, 0.f, 1.f);
            if (GEOM) ge = geo_lds[j];
            const float w = (j < cnt) ? pair_basis<BASIS>(g, lb, (int64_t)cb + j, ge.x, ge.y, ge.z, ge.w) : 0.0f;
            w_lds[j][k] = w;
        }
        __syncthreads();
        if (want_df) {
            for (int j0 = 0; j0 < cnt; j0 += GF) {
                const int j = j0 + slot;
                if (j < cnt && fvalid) {
                    float gf = 0.0f;
#pragma unroll
                    for (int q = 0; q < KPAD; q += 4) {
                        const float4 wv = *(const float4 *)&w_lds[j][q];
                        gf += gp[q] * wv.x + gp[q + 1] * wv.y + gp[q + 2] * wv.z + gp[q + 3] * wv.w;
                    }
                    if (g.deterministic) feat_grads[(int64_t)(cb + j) * g.c_in + f] = gf;
                    else unsafeAtomicAdd(&feat_grads[(int64_t)nidx_lds[j] * g.c_in + f], gf);
                }
            }
        }
        if (want_db) {
            for (int j0 = 0; j0 < cnt; j0 += PARTS) {
                const int j = j0 + part;
                if (j < cnt) {
                    float acc = 0.0f;
#pragma unroll
                    for (int q = 0; q < FPAD; q += 4) {
                        const float4 rv = *(const float4 *)&row_lds[j][q];
                        acc += gt[q] * rv.x + gt[q + 1] * rv.y + gt[q + 2] * rv.z + gt[q + 3] * rv.w;
                    }
                    db_lds[j][k] = acc;
                }
            }
        }
        __syncthreads();
        if (FUSED) {
            for (int p = 0; p * PARTS < cnt; ++p) {
                const int j = p * PARTS + part;
                const float4 ge = geo_lds[j];
                float gx = 0.f, gy = 0.f, gz = 0.f, gpdf = 0.f;
                if (j < cnt && lb.active)
                    basis_derivative<BASIS>(g, lb, ge.x, ge.y, ge.z, ge.w, db_lds[j][k], gx, gy, gz, gpdf, p0, p1, p2, p3);
                if (!geometry) continue;                // only the parameters' gradients are asked for
                // summed over the basis index: the KPAD lanes of this pair
                gx = pccnn_group_sum<KPAD>(gx);
                gy = pccnn_group_sum<KPAD>(gy);
                gz = pccnn_group_sum<KPAD>(gz);
                if (BasisTraits<BASIS>::pdf_grad) gpdf = pccnn_group_sum<KPAD>(gpdf);
                if (k < 4) g_lds[j][k] = (k == 0) ? gx * ir0 : (k == 1) ? gy * ir1 : (k == 2) ? gz * ir2 : gpdf;
            }
            __syncthreads();
            for (int i = 0; geometry && i * 16 < cnt; ++i) {
                const int j = i * 16 + (lane >> 2), comp = lane & 3;
                if (j < cnt) {
                    const int jn = nidx_lds[j];
                    const float v = g_lds[j][comp];
                    if (comp < 3) sg += v;
                    if (pair_grads) {
                        // per-pair values, summed per point afterwards by conv_point_gather_kernel
                        pair_grads[(int64_t)(cb + j) * 4 + comp] = v;
                    } else if (comp < 3) {
                        if (d_pts) unsafeAtomicAdd(&d_pts[(int64_t)jn * 3 + comp], v);
                    } else if (BasisTraits<BASIS>::pdf_grad && d_pdf) {
                        unsafeAtomicAdd(&d_pdf[jn], v);
                    }
                }
            }
        } else if (want_db) {
            for (int idx = lane; idx < cnt * KPAD; idx += 64) {
                const int j = idx / KPAD, kk = idx % KPAD;
                if (kk < g.k) basis_grads[(int64_t)(cb + j) * g.k + kk] = db_lds[j][kk];
            }
        }
        __syncthreads();
    }
    if (FUSED) {
        sg = pccnn_strided_sum<4>(sg);
        if (lane < 3 && d_samples) d_samples[s * 3 + lane] = -sg;
        if (param_partials) {
            p0 = pccnn_strided_sum<KPAD>(p0);
            p1 = pccnn_strided_sum<KPAD>(p1);
            p2 = pccnn_strided_sum<KPAD>(p2);
            if (BasisTraits<BASIS>::axis) p3 = pccnn_strided_sum<KPAD>(p3);
            constexpr int COMPS = BasisTraits<BASIS>::axis ? 4 : 3;
            if (g.deterministic) {
                float *prow = param_partials + s * (4 * KPAD);
                for (int c = part; c < 4; c += PARTS)
                    prow[c * KPAD + k] = (c == 0) ? p0 : (c == 1) ? p1 : (c == 2) ? p2 : (COMPS == 4 ? p3 : 0.0f);
            } else {
                float *prow = param_partials + (int64_t)(blockIdx.x % PARAM_ROWS) * 256;
                for (int c = part; c < COMPS; c += PARTS) {
                    const float v = (c == 0) ? p0 : (c == 1) ? p1 : (c == 2) ? p2 : p3;
                    unsafeAtomicAdd(&prow[c * 64 + k], v);
                }
            }
        }
    }
}

// Symmetric neighborhoods (samples are the points, uncapped search): pair (a, b) exists iff (b, a) does.
// mirror[t] of pair t = (point a, sample b) is the index of pair (point b, sample a), found by scanning
// sample a's segment; -1 and a count in *missing when there is none (the neighborhood is not symmetric).
__global__ void __launch_bounds__(256)
mirror_pairs_kernel(const int2 *__restrict__ neigh, const int32_t *__restrict__ ends, int64_t t, int64_t m,
                    int32_t *__restrict__ mirror, int32_t *__restrict__ missing)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= t) return;
    const int2 pr = neigh[i];
    int found = -1;
    if (pr.x >= 0 && pr.x < m) {
        const int lo = pr.x > 0 ? ends[pr.x - 1] : 0, hi = ends[pr.x];
        for (int j = lo; j < hi; ++j)
            if (neigh[j].x == pr.y) { found = j; break; }
    }
    mirror[i] = found;
    if (found < 0) atomicAdd(missing, 1);
}

// d_pts[n] and d_pdf[n] of a symmetric neighborhood: the pairs in which n is the point are the mirrors of
// the pairs of sample n.  Four lanes per point: lane q adds the (x, y, z, density) records of the pairs
// q, q + 4, ... of the segment (16-byte loads, independent between the lanes), two exchanges add the four
// partial sums in a fixed order, and lane q stores component q.
// The pairs of point n are listed in index[lo .. hi): with `starts` == 0 the bounds are the segment of sample n in
// `bounds` (running totals, the layout of `ends`: the index is the mirror index of a symmetric neighborhood); with
// `starts` != 0 they are bounds[n] and bounds[n + 1] (the by-point index of conv_by_point_index).
__device__ __forceinline__ void point_segment(const int32_t *__restrict__ bounds, int starts, int64_t n, int &lo, int &hi)
{
    if (starts) { lo = bounds[n]; hi = bounds[n + 1]; }
    else { lo = n > 0 ? bounds[n - 1] : 0; hi = bounds[n]; }
}

__global__ void __launch_bounds__(256)
conv_point_gather_kernel(const float *__restrict__ pair_grads, const int32_t *__restrict__ mirror,
                         const int32_t *__restrict__ ends, int starts, int64_t m, float *__restrict__ d_pts,
                         float *__restrict__ d_pdf)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t n = i >> 2;
    const int q = (int)(i & 3);
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (n < m) {
        int lo, hi;
        point_segment(ends, starts, n, lo, hi);
        const float4 *rec = (const float4 *)pair_grads;
        for (int j = lo + q; j < hi; j += 4) {
            const float4 v = rec[mirror[j]];
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
    }
#pragma unroll
    for (int o = 1; o < 4; o <<= 1) {
        acc.x += __shfl_xor(acc.x, o);
        acc.y += __shfl_xor(acc.y, o);
        acc.z += __shfl_xor(acc.z, o);
        acc.w += __shfl_xor(acc.w, o);
    }
    if (n >= m) return;
    const float v = (q == 0) ? acc.x : (q == 1) ? acc.y : (q == 2) ? acc.z : acc.w;
    if (q < 3) {
        if (d_pts) d_pts[n * 3 + q] = v;
    } else if (d_pdf) {
        d_pdf[n] = v;
    }
}

// d_feats[n][:] = sum of the per-pair rows rows[index[j]][:] over the pairs j of point n (bounds as in
// conv_point_gather_kernel), in the order of the index: the feature gradients without atomics.  LANES lanes per
// point (the row width rounded up to a power of two, at most 64); wider rows in blocks of 64 features.
template <int LANES>
__global__ void __launch_bounds__(256)
conv_rows_gather_kernel(const float *__restrict__ rows, const int32_t *__restrict__ index,
                        const int32_t *__restrict__ bounds, int starts, int64_t n_points, int c_in,
                        float *__restrict__ d_feats)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n = i / LANES;
    const int l = (int)(i % LANES);
    if (n >= n_points) return;
    int lo, hi;
    point_segment(bounds, starts, n, lo, hi);
    for (int f = l; f < c_in; f += LANES) {
        float acc = 0.0f;
        int j = lo;
        for (; j + 4 <= hi; j += 4) {
            const float v0 = rows[(int64_t)index[j] * c_in + f], v1 = rows[(int64_t)index[j + 1] * c_in + f];
            const float v2 = rows[(int64_t)index[j + 2] * c_in + f], v3 = rows[(int64_t)index[j + 3] * c_in + f];
            acc += v0;
            acc += v1;
            acc += v2;
            acc += v3;
        }
        for (; j < hi; ++j) acc += rows[(int64_t)index[j] * c_in + f];
        d_feats[n * c_in + f] = acc;
    }
}

__global__ void __launch_bounds__(256)
pair_point_keys_kernel(const int2 *__restrict__ neigh, int64_t t, int64_t *__restrict__ keys)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < t) keys[i] = neigh[i].x;
}

// The pair list by point, for a neighborhood without a mirror index: order_out i32[t] lists the pairs sorted by
// their point (pairs of one point in ascending pair index: the sort is stable), starts_out i32[n + 1] the first
// entry of every point.  Workspace: two i64[t] key arrays and the sort's own.
static size_t by_point_index_bytes(int64_t n, int64_t t)
{
    return 2 * pccnn_align((size_t)t * sizeof(int64_t)) + pccnn_align(pccnn_sort_keys_workspace_bytes(t)) +
           pccnn_align((size_t)t * sizeof(int32_t)) + pccnn_align(((size_t)n + 1) * sizeof(int32_t));
}

static int conv_by_point_index(const int2 *neigh, int64_t n, int64_t t, int32_t *order_out, int32_t *starts_out,
                               PccnnArena &arena, hipStream_t s)
{
    int64_t *keys = arena.take<int64_t>((size_t)t);
    int64_t *sorted = arena.take<int64_t>((size_t)t);
    const size_t sort_bytes = pccnn_sort_keys_workspace_bytes(t);
    void *sort_ws = arena.take<char>(sort_bytes);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv backward: workspace too small for the by-point pair index");
    pair_point_keys_kernel<<<(unsigned)pccnn_ceil_div(t, 256), 256, 0, s>>>(neigh, t, keys);
    PCCNN_LAUNCH_CHECK();
    int bits = 1;
    while (bits < 62 && (1ll << bits) < n) ++bits;
    int rc = pccnn_sort_keys(keys, t, bits, sorted, order_out, nullptr, 3, nullptr, sort_ws, sort_bytes, s);
    if (rc != PCCNN_OK) return rc;
    return pccnn_build_cell_table(sorted, t, n, starts_out, s);
}

// Sums partial rows ([rows][256], column = component * 64 + basis index) in a fixed order.
// Stage 1: workgroup b adds the rows b, b + G, b + 2G, ... (thread = column, coalesced); stage 2: one
// workgroup adds the G stage-1 rows and writes every value to its place in the parameter gradient tensors.
#define PARAM_REDUCE_GROUPS 64
#define PARAM_REDUCE_GROUPS_PER_SAMPLE 128      // first-stage groups when every sample wrote a partial row

__global__ void __launch_bounds__(256)
conv_param_reduce1_kernel(const float *__restrict__ partials, int64_t rows, float *__restrict__ stage)
{
    float acc = 0.0f;
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) acc += partials[r * 256 + threadIdx.x];
    stage[(int64_t)blockIdx.x * 256 + threadIdx.x] = acc;
}

// The same first stage over compact per-sample rows [4][kpad] (the pass without atomics): column c * 64 + k of the
// stage row comes from entry c * kpad + k.  Workgroup b sums a contiguous run of rows; its 256 threads cover
// 256 / (4 kpad) rows at a time (thread = (row lane, entry)), eight loads in flight each, and the row lanes meet in
// LDS - a fixed order throughout.
__global__ void __launch_bounds__(256)
conv_param_reduce1_compact_kernel(const float *__restrict__ partials, int64_t rows, int kpad, float *__restrict__ stage)
{
    __shared__ float part[256];
    const int width = 4 * kpad;                         // 32 .. 256 entries per row
    const int lanes = 256 / width;
    const int col = threadIdx.x % width, lane = threadIdx.x / width;
    const int64_t per = (rows + gridDim.x - 1) / gridDim.x;
    const int64_t r0 = (int64_t)blockIdx.x * per;
    const int64_t r1 = r0 + per < rows ? r0 + per : rows;
    float acc = 0.0f;
    int64_t r = r0 + lane;
    for (; r + 7 * lanes < r1; r += 8 * lanes) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = partials[(r + (int64_t)u * lanes) * width + col];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; r < r1; r += lanes) acc += partials[r * width + col];
    part[threadIdx.x] = acc;
    __syncthreads();
    // thread t writes stage column t = c * 64 + k
    const int c = threadIdx.x >> 6, k = threadIdx.x & 63;
    float total = 0.0f;
    if (k < kpad)
        for (int l = 0; l < lanes; ++l) total += part[l * width + c * kpad + k];
    stage[(int64_t)blockIdx.x * 256 + threadIdx.x] = total;
}

template <int BASIS>
__global__ void __launch_bounds__(256)
conv_param_reduce2_kernel(const float *__restrict__ stage, int groups, int k_basis, float *__restrict__ dst_a,
                          float *__restrict__ dst_b)
{
    const int comp = threadIdx.x >> 6, kk = threadIdx.x & 63;
    float acc = 0.0f;
    int r = 0;
    for (; r + 8 <= groups; r += 8) {                   // eight loads in flight, added in order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = stage[(r + u) * 256 + threadIdx.x];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; r < groups; ++r) acc += stage[r * 256 + threadIdx.x];
    if (kk < k_basis && dst_a) {
        if (BasisTraits<BASIS>::kernel_pts) {
            if (comp < 3) dst_a[kk * 3 + comp] = acc;               // d_kernel_pts [K,3]
        } else {
            if (comp < 3) dst_a[comp * k_basis + kk] = acc;         // d_axis [3,K]
            else dst_b[kk] = acc;                                   // d_bias [K]
        }
    }
}

// Variance statistic of the initialisation: per sample, sum over ordered neighbor pairs (i, j) of
// (w_i . w_j)(F_i . F_j) = the squared Frobenius norm of the sample's projection tile P[s].  One wavefront
// per row of P sums the squares; one workgroup then forms 1 / mean over the samples in double, fixed order.
__global__ void __launch_bounds__(256)
row_sumsq_kernel(const float *__restrict__ proj, int64_t rows, int64_t row_len, float *__restrict__ out)
{
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const float *src = proj + r * row_len;
    float acc = 0.0f;
    for (int64_t i = pccnn_lane(); i < row_len; i += 64) acc += src[i] * src[i];
    acc = pccnn_wave_sum(acc);
    if (pccnn_lane() == 0) out[r] = acc;
}

__global__ void __launch_bounds__(256)
mean_reciprocal_kernel(const float *__restrict__ vals, int64_t count, float *__restrict__ out)
{
    __shared__ double red[256];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += 256) acc += (double)vals[i];
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if (threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = (float)(1.0 / (red[0] / (double)count));
}

// out[s][c] = in[s][c] / (number of neighbors of s + 1e-6): the SPHConv normalisation.
__global__ void __launch_bounds__(256)
scale_by_count_kernel(const float *__restrict__ in, float *__restrict__ out, const int32_t *__restrict__ ends,
                      int64_t m, int c_out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= m * c_out) return;
    const int64_t s = i / c_out;
    const float cnt = (float)(ends[s] - (s > 0 ? ends[s - 1] : 0));
    out[i] = in[i] / (cnt + 1e-6f);
}

// Squared row norms divided by the squared neighbor count (weight variance with division).
__global__ void __launch_bounds__(256)
divide_by_count_sq_kernel(float *__restrict__ rows, const int32_t *__restrict__ ends, int64_t m)
{
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= m) return;
    const int cnt = ends[s] - (s > 0 ? ends[s - 1] : 0);
    const float inv = cnt > 0 ? 1.0f / (float)cnt : 0.0f;
    rows[s] = rows[s] * inv * inv;
}

// PointConv's own basis op: basis[t][k] = d_t . A[:,k] + b[k], one thread per (pair, k).
__global__ void __launch_bounds__(256)
linear_basis_fwd_kernel(ConvGeom g, float *__restrict__ basis_out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= g.t * g.k) return;
    const int64_t t = i / g.k;
    const int k = (int)(i % g.k);
    const int2 pr = g.neigh[t];
    const float dx = (g.pts[(int64_t)pr.x * 3 + 0] - g.samples[(int64_t)pr.y * 3 + 0]) * (1.0f / g.radii[0]);
    const float dy = (g.pts[(int64_t)pr.x * 3 + 1] - g.samples[(int64_t)pr.y * 3 + 1]) * (1.0f / g.radii[1]);
    const float dz = (g.pts[(int64_t)pr.x * 3 + 2] - g.samples[(int64_t)pr.y * 3 + 2]) * (1.0f / g.radii[2]);
    basis_out[i] = dx * g.basis_a[k] + dy * g.basis_a[g.k + k] + dz * g.basis_a[2 * g.k + k] + g.basis_b[k];
}

// Its backward, pair-parallel (the op gets no segment offsets): KPAD lanes per pair as in
// conv_basis_bwd_kernel, float atomics for the point and the sample gradients.
template <int KPAD>
__global__ void __launch_bounds__(256)
linear_basis_bwd_kernel(ConvGeom g, const float *__restrict__ basis_grads, float *__restrict__ d_pts,
                        float *__restrict__ d_samples, float *__restrict__ param_partials)
{
    __shared__ float lds_param[4][4 * 64];
    constexpr int PAIRS = 64 / KPAD;
    const int lane = pccnn_lane(), wave = threadIdx.x >> 6;
    const int k = lane % KPAD, sub = lane / KPAD;
    const bool kvalid = k < g.k;
    const float ir0 = 1.0f / g.radii[0], ir1 = 1.0f / g.radii[1], ir2 = 1.0f / g.radii[2];
    float c0 = 0.f, c1 = 0.f, c2 = 0.f;
    if (kvalid) { c0 = g.basis_a[k]; c1 = g.basis_a[g.k + k]; c2 = g.basis_a[2 * g.k + k]; }
    float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
    const int64_t gw = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t nw = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t base = gw * PAIRS; base < g.t; base += nw * PAIRS) {
        const int64_t t = base + sub;
        const bool tv = t < g.t;
        float gx = 0.f, gy = 0.f, gz = 0.f;
        int2 pr = make_int2(0, 0);
        if (tv) {
            pr = g.neigh[t];
            if (kvalid) {
                const float dx = (g.pts[(int64_t)pr.x * 3 + 0] - g.samples[(int64_t)pr.y * 3 + 0]) * ir0;
                const float dy = (g.pts[(int64_t)pr.x * 3 + 1] - g.samples[(int64_t)pr.y * 3 + 1]) * ir1;
                const float dz = (g.pts[(int64_t)pr.x * 3 + 2] - g.samples[(int64_t)pr.y * 3 + 2]) * ir2;
                const float c = basis_grads[t * g.k + k];
                gx = c * c0; gy = c * c1; gz = c * c2;
                p0 += dx * c; p1 += dy * c; p2 += dz * c; p3 += c;
            }
        }
#pragma unroll
        for (int o = KPAD / 2; o > 0; o >>= 1) {
            gx += __shfl_xor(gx, o);
            gy += __shfl_xor(gy, o);
            gz += __shfl_xor(gz, o);
        }
        if (tv && k == 0) {
            gx *= ir0; gy *= ir1; gz *= ir2;
            unsafeAtomicAdd(&d_pts[(int64_t)pr.x * 3 + 0], gx);
            unsafeAtomicAdd(&d_pts[(int64_t)pr.x * 3 + 1], gy);
            unsafeAtomicAdd(&d_pts[(int64_t)pr.x * 3 + 2], gz);
            unsafeAtomicAdd(&d_samples[(int64_t)pr.y * 3 + 0], -gx);
            unsafeAtomicAdd(&d_samples[(int64_t)pr.y * 3 + 1], -gy);
            unsafeAtomicAdd(&d_samples[(int64_t)pr.y * 3 + 2], -gz);
        }
    }
#pragma unroll
    for (int o = KPAD; o < 64; o <<= 1) {
        p0 += __shfl_xor(p0, o);
        p1 += __shfl_xor(p1, o);
        p2 += __shfl_xor(p2, o);
        p3 += __shfl_xor(p3, o);
    }
    if (sub == 0) {
        lds_param[wave][k] = p0;
        lds_param[wave][64 + k] = p1;
        lds_param[wave][128 + k] = p2;
        lds_param[wave][192 + k] = p3;
    }
    __syncthreads();
    const int i = threadIdx.x, comp = i >> 6, kk = i & 63;
    float v = 0.0f;
    if (kk < KPAD) v = lds_param[0][comp * 64 + kk] + lds_param[1][comp * 64 + kk] + lds_param[2][comp * 64 + kk] +
                       lds_param[3][comp * 64 + kk];
    param_partials[(int64_t)blockIdx.x * 256 + i] = v;
}

// ------------------------------------------------------------------------------- host side

static int kpad_of(int k) { return k <= 8 ? 8 : (k <= 16 ? 16 : (k <= 32 ? 32 : 64)); }

// `bf16`: proj is uint16_t[m, c_in * k] of bf16 bit patterns instead of float[m, c_in * k].
template <int BASIS, int KPAD>
static void launch_proj_fwd_narrow(const ConvGeom &g, const float *feats, void *proj, hipStream_t s, bool bf16)
{
    dim3 grid(conv_sample_blocks(g.m));
#define NARROW_GO(FP)                                                                                   \
    do {                                                                                                \
        if (bf16) conv_proj_fwd_narrow_kernel<BASIS, KPAD, FP, true><<<grid, 64, 0, s>>>(g, feats, proj);  \
        else conv_proj_fwd_narrow_kernel<BASIS, KPAD, FP, false><<<grid, 64, 0, s>>>(g, feats, proj);      \
    } while (0)
    if (g.c_in <= 8) NARROW_GO(8);
    else if (g.c_in <= 16) NARROW_GO(16);
    else NARROW_GO(32);
#undef NARROW_GO
}

template <int BASIS>
static int launch_proj_fwd(const ConvGeom &g, const float *feats, void *proj, hipStream_t s, bool bf16 = false)
{
    dim3 grid(conv_sample_blocks(g.m), (unsigned)((g.c_in + 63) / 64));
    PccnnTimed timed(PCCNN_T_PROJ_FWD, s);
    if (g.c_in <= 32) {
        // few input features: several pairs side by side instead of idle lanes
        switch (kpad_of(g.k)) {
        case 8: launch_proj_fwd_narrow<BASIS, 8>(g, feats, proj, s, bf16); break;
        case 16: launch_proj_fwd_narrow<BASIS, 16>(g, feats, proj, s, bf16); break;
        case 32: launch_proj_fwd_narrow<BASIS, 32>(g, feats, proj, s, bf16); break;
        default: launch_proj_fwd_narrow<BASIS, 64>(g, feats, proj, s, bf16); break;
        }
        PCCNN_LAUNCH_CHECK();
        return PCCNN_OK;
    }
#define PROJ_GO(KP)                                                                         \
    do {                                                                                    \
        if (bf16) conv_proj_fwd_kernel<BASIS, KP, true><<<grid, 64, 0, s>>>(g, feats, proj);  \
        else conv_proj_fwd_kernel<BASIS, KP, false><<<grid, 64, 0, s>>>(g, feats, proj);      \
    } while (0)
    switch (kpad_of(g.k)) {
    case 8: PROJ_GO(8); break;
    case 16: PROJ_GO(16); break;
    case 32: PROJ_GO(32); break;
    default: PROJ_GO(64); break;
    }
#undef PROJ_GO
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// Where the basis stage of the backward kernel puts its results; members a call does not want are null.
struct BasisGradOut {
    float *basis_grads;     // [t,k], EXPLICIT only
    float *d_pts, *d_samples, *d_pdf;
    float *partials;        // [PARAM_ROWS][256], zeroed by the caller
    float *pair_grads;      // [t][4] per-pair (x, y, z, density) values instead of atomics on d_pts / d_pdf
};

template <int BASIS, int KPAD>
static void launch_proj_bwd_k(const ConvGeom &g, const float *feats, const float *proj_grads, float *feat_grads,
                              bool want_basis, const BasisGradOut &o, hipStream_t s)
{
    dim3 grid(conv_sample_blocks(g.m));
    if (g.c_in <= 32) {
        // few input features: several pairs side by side instead of idle lanes
#define NARROW_GO(FP)                                                                                                  \
    do {                                                                                                               \
        if (feat_grads && want_basis)                                                                                  \
            conv_proj_bwd_narrow_kernel<BASIS, KPAD, FP, true, true><<<grid, 64, 0, s>>>(                              \
                g, feats, proj_grads, feat_grads, o.basis_grads, o.d_pts, o.d_samples, o.d_pdf, o.partials, o.pair_grads); \
        else if (feat_grads)                                                                                           \
            conv_proj_bwd_narrow_kernel<BASIS, KPAD, FP, true, false><<<grid, 64, 0, s>>>(                             \
                g, feats, proj_grads, feat_grads, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);               \
        else                                                                                                           \
            conv_proj_bwd_narrow_kernel<BASIS, KPAD, FP, false, true><<<grid, 64, 0, s>>>(                             \
                g, feats, proj_grads, nullptr, o.basis_grads, o.d_pts, o.d_samples, o.d_pdf, o.partials, o.pair_grads); \
    } while (0)
        if (g.c_in <= 8) NARROW_GO(8);
        else if (g.c_in <= 16) NARROW_GO(16);
        else NARROW_GO(32);
#undef NARROW_GO
        return;
    }
    if (feat_grads && want_basis)
        conv_proj_bwd_kernel<BASIS, KPAD, true, true><<<grid, 64, 0, s>>>(g, feats, proj_grads, feat_grads, o.basis_grads,
                                                                          o.d_pts, o.d_samples, o.d_pdf, o.partials,
                                                                          o.pair_grads);
    else if (feat_grads)
        conv_proj_bwd_kernel<BASIS, KPAD, true, false><<<grid, 64, 0, s>>>(g, feats, proj_grads, feat_grads, nullptr,
                                                                           nullptr, nullptr, nullptr, nullptr, nullptr);
    else
        conv_proj_bwd_kernel<BASIS, KPAD, false, true><<<grid, 64, 0, s>>>(g, feats, proj_grads, nullptr, o.basis_grads,
                                                                           o.d_pts, o.d_samples, o.d_pdf, o.partials,
                                                                           o.pair_grads);
}

template <int BASIS>
static int launch_proj_bwd(const ConvGeom &g, const float *feats, const float *proj_grads, float *feat_grads,
                           bool want_basis, const BasisGradOut &o, hipStream_t s)
{
    if (!feat_grads && !want_basis) return PCCNN_OK;
    PccnnTimed timed(PCCNN_T_PROJ_BWD, s);
    switch (kpad_of(g.k)) {
    case 8: launch_proj_bwd_k<BASIS, 8>(g, feats, proj_grads, feat_grads, want_basis, o, s); break;
    case 16: launch_proj_bwd_k<BASIS, 16>(g, feats, proj_grads, feat_grads, want_basis, o, s); break;
    case 32: launch_proj_bwd_k<BASIS, 32>(g, feats, proj_grads, feat_grads, want_basis, o, s); break;
    default: launch_proj_bwd_k<BASIS, 64>(g, feats, proj_grads, feat_grads, want_basis, o, s); break;
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

static int conv_validate(const char *who, int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int num_mlps,
                         int c_out)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED, "%s: d=%d is not supported (2 <= d <= 6)", who, d);
    PCCNN_REQUIRE(n >= 0 && m >= 0 && t >= 0 && n < (1ll << 31) && m < (1ll << 31) && t < (1ll << 31),
                  PCCNN_ERR_INVALID, "%s: n=%lld m=%lld t=%lld", who, (long long)n, (long long)m, (long long)t);
    PCCNN_REQUIRE(c_in >= 1 && c_out >= 1, PCCNN_ERR_INVALID, "%s: c_in=%d c_out=%d", who, c_in, c_out);
    PCCNN_REQUIRE(k >= 1 && k <= 64, PCCNN_ERR_UNSUPPORTED, "%s: basis size k=%d outside [1,64]", who, k);
    PCCNN_REQUIRE(num_mlps >= 1 && c_in % num_mlps == 0 && c_out % num_mlps == 0 && k % num_mlps == 0,
                  PCCNN_ERR_INVALID, "%s: num_mlps=%d must divide c_in=%d, c_out=%d and k=%d", who, num_mlps, c_in,
                  c_out, k);
    return PCCNN_OK;
}

#define CONV_SPLIT_K 64

extern "C" size_t pccnn_conv_workspace_bytes(int64_t m, int64_t t, int c_in, int k, int c_out, int backward)
{
    if (m < 1) m = 1;
    if (t < 1) t = 1;
    size_t proj = pccnn_align((size_t)m * c_in * k * sizeof(float));
    size_t w16 = pccnn_align((size_t)c_in * k * c_out * sizeof(uint16_t));       // bf16 copy of the weights
    size_t pair_b = 2 * pccnn_align((size_t)t * k * sizeof(float));              // basis (+ its gradient) when d != 3
    // (a forward call that keeps no projection may run fused and then needs room for the repacked weights only)
    if (!backward) return proj + w16 + pair_b + pccnn_conv_fused_workspace_bytes(c_in, k, c_out) + 256;
    size_t basis_g = pccnn_align((size_t)t * k * sizeof(float));
    size_t splitk = pccnn_align((size_t)CONV_SPLIT_K * c_in * k * c_out * sizeof(float));
    size_t partials = pccnn_align(((size_t)PARAM_ROWS + PARAM_REDUCE_GROUPS) * 256 * sizeof(float));
    size_t scaled = pccnn_align((size_t)m * c_out * sizeof(float));
    size_t pair_g = pccnn_align((size_t)t * 4 * sizeof(float));
    size_t g16 = pccnn_align((size_t)m * c_out * sizeof(uint16_t));               // bf16 copy of the output gradients
    return 2 * proj + basis_g + splitk + partials + scaled + pair_g + w16 + g16 + pair_b + 256;
}

extern "C" size_t pccnn_conv_workspace_bytes_deterministic(int64_t n, int64_t m, int64_t t, int c_in, int k, int c_out)
{
    if (n < 1) n = 1;
    if (m < 1) m = 1;
    if (t < 1) t = 1;
    return pccnn_conv_workspace_bytes(m, t, c_in, k, c_out, 1) +
           pccnn_align(((size_t)m + PARAM_REDUCE_GROUPS_PER_SAMPLE) * 256 * sizeof(float)) +
           pccnn_align((size_t)t * c_in * sizeof(float)) + by_point_index_bytes(n, t) + 256;
}

// out[m, c_out] = P[m, c_in*k] x W, with the feature axis split over num_mlps independent
// weight blocks (num_mlps == 1 is the plain product).
// Split of the sample dimension for d_weights = P^T x dOut, whose output ([K*Cin, Cout]) has few tiles: enough
// workgroups for about four per CU, but (fp32 operands) at least 2048 samples each, so that the partial sums
// written and summed again stay small beside the product itself.
static int conv_split_k(int64_t inner, int64_t co, int num_mlps, int64_t m, bool bf16)
{
    if (m < 4096) return 1;
    if (bf16) return CONV_SPLIT_K;      // bound by its operand traffic: the more workgroups in flight the better
    const int64_t tiles = pccnn_ceil_div(inner, 64) * pccnn_ceil_div(co, 128) * num_mlps;
    int64_t split = 1024 / tiles;
    if (split > m / 2048) split = m / 2048;
    if (split > CONV_SPLIT_K) split = CONV_SPLIT_K;
    return (int)(split < 1 ? 1 : split);
}

static int contraction_fwd(const float *proj, const float *weights, float *out, int64_t m, int c_in, int k,
                           int num_mlps, int c_out, hipStream_t s)
{
    const int64_t inner = (int64_t)c_in * k / num_mlps;
    const int64_t co = c_out / num_mlps;
    return pccnn_gemm_f32(proj, weights, out, m, co, inner, 0, 0, (int64_t)c_in * k, co, c_out, num_mlps, inner,
                          inner * co, co, 1, nullptr, 0, s);
}

// `bf16`: the projection (proj_out, when given, is uint16_t[m, c_in * k]) and a copy of the weights are kept as
// bf16 and contracted on the bf16 matrix pipe with fp32 accumulation; everything else stays fp32.
template <int BASIS>
static int conv_forward(ConvGeom g, const float *feats, const float *weights, int num_mlps, int c_out, float *out,
                        void *proj_out, void *workspace, size_t workspace_bytes, hipStream_t s,
                        bool divide_by_count = false, bool bf16 = false)
{
    if (g.m == 0) return PCCNN_OK;
    if constexpr (BASIS != BASIS_SPH) {
        // nobody wants the projection: it stays on chip, slice by slice, between the gather and the matrix cores
        if (proj_out == nullptr && pccnn_conv_fused_eligible(BASIS, g.c_in, g.k, num_mlps, c_out)) {
            PCCNN_REQUIRE(workspace && workspace_bytes >= pccnn_conv_fused_workspace_bytes(g.c_in, g.k, c_out),
                          PCCNN_ERR_WORKSPACE, "conv forward: workspace of %zu bytes, need %zu", workspace_bytes,
                          pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 0));
            return pccnn_conv_fused_forward<BASIS>(g, feats, weights, c_out, out, workspace, divide_by_count, bf16, s);
        }
    }
    PccnnArena arena(workspace, workspace_bytes);
    void *proj = proj_out;
    if (proj == nullptr) proj = arena.take<float>((size_t)g.m * g.c_in * g.k);
    const int64_t w_count = (int64_t)g.c_in * g.k * c_out / num_mlps;
    uint16_t *w16 = bf16 ? arena.take<uint16_t>((size_t)w_count) : nullptr;
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv forward: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 0));
    int rc = launch_proj_fwd<BASIS>(g, feats, proj, s, bf16);
    if (rc != PCCNN_OK) return rc;
    if (bf16) {
        const int64_t inner = (int64_t)g.c_in * g.k / num_mlps;
        const int64_t co = c_out / num_mlps;
        if ((rc = pccnn_f32_to_bf16(weights, w16, w_count, s)) != PCCNN_OK) return rc;
        rc = pccnn_gemm_bf16((const uint16_t *)proj, w16, out, g.m, co, inner, 0, 0, (int64_t)g.c_in * g.k, co, c_out,
                             num_mlps, inner, inner * co, co, 1, nullptr, 0, s);
    } else {
        rc = contraction_fwd((const float *)proj, weights, out, g.m, g.c_in, g.k, num_mlps, c_out, s);
    }
    if (rc != PCCNN_OK || !divide_by_count) return rc;
    scale_by_count_kernel<<<(unsigned)pccnn_ceil_div(g.m * c_out, 256), 256, 0, s>>>(out, out, g.ends, g.m, c_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// What the backward call does before its contractions, in one launch: the accumulators that the projection kernel
// adds into are cleared and the bf16 copies of the output gradients and of the weights are made (up to four
// arrays to clear and two to convert; unused entries have a count of zero).  One thread per four elements of the
// jobs laid end to end.
struct ConvPrepJobs {
    float *zero[4];
    int64_t zero_count[4];
    const float *src[2];
    uint16_t *dst[2];
    int64_t convert_count[2];
};

__global__ void __launch_bounds__(256) conv_prep_kernel(ConvPrepJobs jobs, int64_t quads)
{
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (int64_t)gridDim.x * blockDim.x) {
        int64_t at = q;
        bool done = false;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t job_quads = (jobs.zero_count[j] + 3) / 4;
            if (!done && at < job_quads) {
                float *p = jobs.zero[j] + at * 4;
                const int64_t left = jobs.zero_count[j] - at * 4;
                if (left >= 4 && (((uintptr_t)p) & 15) == 0) {
                    *(float4 *)p = make_float4(0.f, 0.f, 0.f, 0.f);
                } else {
                    for (int e = 0; e < 4 && e < left; ++e) p[e] = 0.0f;
                }
                done = true;
            }
            if (!done) at -= job_quads;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t job_quads = (jobs.convert_count[j] + 3) / 4;
            if (!done && at < job_quads) {
                const int64_t left = jobs.convert_count[j] - at * 4;
                for (int e = 0; e < 4 && e < left; ++e) jobs.dst[j][at * 4 + e] = pccnn_bf16_bits(jobs.src[j][at * 4 + e]);
                done = true;
            }
            if (!done) at -= job_quads;
        }
    }
}

static int conv_prep(const ConvPrepJobs &jobs, hipStream_t s)
{
    int64_t quads = 0;
    for (int j = 0; j < 4; ++j) quads += (jobs.zero_count[j] + 3) / 4;
    for (int j = 0; j < 2; ++j) quads += (jobs.convert_count[j] + 3) / 4;
    if (quads == 0) return PCCNN_OK;
    int64_t blocks = pccnn_ceil_div(quads, 256);
    if (blocks > 16384) blocks = 16384;
    conv_prep_kernel<<<(unsigned)blocks, 256, 0, s>>>(jobs, quads);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// Gradients are produced only for the groups named in `mask`; pointers of groups not requested may be null.
template <int BASIS>
static int conv_backward(ConvGeom g, const float *feats, const float *weights, const float *in_grads, int num_mlps,
                         int c_out, const void *proj_in, int mask, float *d_weights, float *d_feats,
                         float *d_param_a, float *d_param_b, float *d_pdf, float *d_pts, float *d_samples,
                         void *workspace, size_t workspace_bytes, hipStream_t s, bool divide_by_count = false,
                         const int32_t *mirror = nullptr, bool bf16 = false)
{
    // bf16: proj_in (when given) is uint16_t[m, c_in * k]; the two contractions take bf16 copies of the weights
    // and of the output gradients, accumulate in fp32 and return fp32 (d_weights, d_proj)
    // d_param_a: d_kernel_pts [K,3] (kernel-point families), d_axis [3,K] (MLP) or the per-pair basis
    // gradient [T,K] (EXPLICIT); d_param_b: d_bias [K] (MLP only)
    typedef BasisTraits<BASIS> Tr;
    const int64_t count_a = (BASIS == BASIS_EXPLICIT) ? g.t * g.k : 3 * g.k;
    const int count_b = (BASIS == BASIS_MLP ? g.k : 0);
    const bool want_w = mask & PCCNN_GRAD_WEIGHTS, want_f = mask & PCCNN_GRAD_FEATS;
    const bool want_par = (mask & PCCNN_GRAD_BASIS_PARAMS) && (Tr::differentiable || BASIS == BASIS_EXPLICIT);
    const bool want_pts = (mask & PCCNN_GRAD_PTS) && Tr::differentiable;
    const bool want_pdf = (mask & PCCNN_GRAD_PDF) && Tr::pdf_grad;
    const bool want_basis = want_par || want_pts || want_pdf;
    int rc;
    // PCCNN_GRAD_DETERMINISTIC: no float atomics anywhere in the pass.  Feature gradients go to one row per pair
    // and are summed per point in the order of the mirror index (symmetric neighborhoods) or of a by-point index of
    // the pair list built here; the point-side gradients take the same route; every sample writes its own
    // basis-parameter partial row.
    const bool det = (mask & PCCNN_GRAD_DETERMINISTIC) != 0 && g.m > 0 && g.t > 0;
    // The per-pair rows and their gather are also the faster way to the feature gradients when they are all the
    // projection pass has to produce, the rows are wide and a mirror index is at hand (65 536 samples, 0.92 M pairs,
    // 64 features: feature + weight gradients in 480 instead of 512 us); taken when the workspace has the room.
    const bool rows_auto = !det && mirror != nullptr && want_f && !want_basis && g.c_in > 32 && g.m > 0 && g.t > 0 &&
                           workspace_bytes >= pccnn_conv_workspace_bytes_deterministic(g.n, g.m, g.t, g.c_in, g.k, c_out);
    const bool rows_route = det || rows_auto;
    g.deterministic = rows_route ? 1 : 0;
    PccnnArena arena(workspace, workspace_bytes);
    const int64_t partial_rows = det ? g.m : PARAM_ROWS;
    const int reduce_groups = det ? PARAM_REDUCE_GROUPS_PER_SAMPLE : PARAM_REDUCE_GROUPS;
    float *partials = arena.take<float>((size_t)(partial_rows + reduce_groups) * 256);
    float *stage = partials + partial_rows * 256;
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv backward: workspace of %zu bytes, need %zu", workspace_bytes,
                  det ? pccnn_conv_workspace_bytes_deterministic(g.n, g.m, g.t, g.c_in, g.k, c_out)
                      : pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 1));
    // with a mirror index (or, in the deterministic pass, the by-point index) the point-side gradients are
    // written once per point, not accumulated
    const bool gather = (mirror != nullptr || det) && Tr::differentiable && (want_pts || want_pdf) && g.m > 0 && g.t > 0;
    // the accumulators to clear; the launch follows below, together with the bf16 copies
    ConvPrepJobs prep = {};
    if (want_f && !rows_route) { prep.zero[0] = d_feats; prep.zero_count[0] = g.n * g.c_in; }
    if (want_pts && !gather) { prep.zero[1] = d_pts; prep.zero_count[1] = g.n * 3; }
    if (want_pdf && !gather) { prep.zero[2] = d_pdf; prep.zero_count[2] = g.n; }
    if (g.m == 0 || g.t == 0) {
        if ((rc = conv_prep(prep, s)) != PCCNN_OK) return rc;
        if (want_pts && (rc = pccnn_fill_f32(d_samples, 0.0f, g.m * 3, s)) != PCCNN_OK) return rc;
        if (want_par && (rc = pccnn_fill_f32(d_param_a, 0.0f, count_a, s)) != PCCNN_OK) return rc;
        if (want_par && count_b && (rc = pccnn_fill_f32(d_param_b, 0.0f, count_b, s)) != PCCNN_OK) return rc;
        if (want_w) return pccnn_fill_f32(d_weights, 0.0f, (int64_t)g.c_in * g.k * c_out / num_mlps, s);
        return PCCNN_OK;
    }

    const size_t proj_elems = (size_t)g.m * g.c_in * g.k;
    float *proj_ws = arena.take<float>(proj_elems);
    float *d_proj = arena.take<float>(proj_elems);
    float *basis_g = arena.take<float>((size_t)g.t * g.k);
    size_t splitk_elems = (size_t)CONV_SPLIT_K * g.c_in * g.k * c_out;
    float *splitk = arena.take<float>(splitk_elems);
    float *scaled_grads = arena.take<float>((size_t)g.m * c_out);
    float *pair_grads = arena.take<float>((size_t)g.t * 4);
    const int64_t w_count = (int64_t)g.c_in * g.k * c_out / num_mlps;
    uint16_t *w16 = bf16 ? arena.take<uint16_t>((size_t)w_count) : nullptr;
    uint16_t *g16 = bf16 ? arena.take<uint16_t>((size_t)g.m * c_out) : nullptr;
    if (BASIS == BASIS_EXPLICIT && want_par) basis_g = d_param_a;    // the basis gradient is itself an output
    // deterministic pass: per-pair feature-gradient rows, and the pairs listed by point
    float *df_rows = (rows_route && want_f) ? arena.take<float>((size_t)g.t * g.c_in) : nullptr;
    const int32_t *by_point = mirror, *by_point_bounds = g.ends;
    int by_point_starts = 0;
    const bool need_index = det && mirror == nullptr && (want_f || gather);
    int32_t *order = need_index ? arena.take<int32_t>((size_t)g.t) : nullptr;
    int32_t *starts = need_index ? arena.take<int32_t>((size_t)g.n + 1) : nullptr;
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv backward: workspace of %zu bytes, need %zu", workspace_bytes,
                  det ? pccnn_conv_workspace_bytes_deterministic(g.n, g.m, g.t, g.c_in, g.k, c_out)
                      : pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 1));
    if (need_index) {
        if ((rc = conv_by_point_index(g.neigh, g.n, g.t, order, starts, arena, s)) != PCCNN_OK) return rc;
        by_point = order;
        by_point_bounds = starts;
        by_point_starts = 1;
    }
    const int64_t inner = (int64_t)g.c_in * g.k / num_mlps;
    const int64_t co = c_out / num_mlps;
    if (divide_by_count) {
        scale_by_count_kernel<<<(unsigned)pccnn_ceil_div(g.m * c_out, 256), 256, 0, s>>>(in_grads, scaled_grads, g.ends,
                                                                                        g.m, c_out);
        PCCNN_LAUNCH_CHECK();
        in_grads = scaled_grads;
    }
    const bool with_projection_pass = want_f || want_basis;
    const bool with_partials = with_projection_pass && want_par && Tr::differentiable;
    // (the deterministic pass stores a partial row per sample instead of adding into shared ones)
    if (with_partials && !det) { prep.zero[3] = partials; prep.zero_count[3] = partial_rows * 256; }
    if (bf16) {
        prep.src[0] = in_grads; prep.dst[0] = g16; prep.convert_count[0] = g.m * c_out;
        if (with_projection_pass) { prep.src[1] = weights; prep.dst[1] = w16; prep.convert_count[1] = w_count; }
    }
    if ((rc = conv_prep(prep, s)) != PCCNN_OK) return rc;
    if (want_w) {
        // d_weights = P^T x dOut; P comes from the caller (kept from the forward call) or is rebuilt here
        const void *proj = proj_in;
        if (proj == nullptr) {
            if ((rc = launch_proj_fwd<BASIS>(g, feats, proj_ws, s, bf16)) != PCCNN_OK) return rc;
            proj = proj_ws;
        }
        const int split = conv_split_k(inner, co, num_mlps, g.m, bf16);
        if (bf16)
            rc = pccnn_gemm_bf16((const uint16_t *)proj, g16, d_weights, inner, co, g.m, 1, 0, (int64_t)g.c_in * g.k,
                                 c_out, co, num_mlps, inner, co, inner * co, split, splitk,
                                 splitk_elems * sizeof(float), s);
        else
            rc = pccnn_gemm_f32((const float *)proj, in_grads, d_weights, inner, co, g.m, 1, 0, (int64_t)g.c_in * g.k,
                                c_out, co, num_mlps, inner, co, inner * co, split, splitk,
                                splitk_elems * sizeof(float), s);
        if (rc != PCCNN_OK) return rc;
    }
    if (!want_f && !want_basis) return PCCNN_OK;
    // d_proj = dOut x W^T
    if (bf16) {
        rc = pccnn_gemm_bf16(g16, w16, d_proj, g.m, inner, co, 0, 1, c_out, co, (int64_t)g.c_in * g.k, num_mlps, co,
                             inner * co, inner, 1, nullptr, 0, s);
    } else {
        rc = pccnn_gemm_f32(in_grads, weights, d_proj, g.m, inner, co, 0, 1, c_out, co, (int64_t)g.c_in * g.k, num_mlps,
                            co, inner * co, inner, 1, nullptr, 0, s);
    }
    if (rc != PCCNN_OK) return rc;
    BasisGradOut o = {basis_g, want_pts ? d_pts : nullptr, want_pts ? d_samples : nullptr, want_pdf ? d_pdf : nullptr,
                      (want_par && Tr::differentiable) ? partials : nullptr, gather ? pair_grads : nullptr};
    if ((rc = launch_proj_bwd<BASIS>(g, feats, d_proj, want_f ? (rows_route ? df_rows : d_feats) : nullptr, want_basis, o,
                                     s)) != PCCNN_OK)
        return rc;
    if (rows_route && want_f) {
        const int lanes = g.c_in <= 8 ? 8 : (g.c_in <= 16 ? 16 : (g.c_in <= 32 ? 32 : 64));
        const unsigned blocks = (unsigned)pccnn_ceil_div(g.n * lanes, 256);
#define ROWS_GO(L) conv_rows_gather_kernel<L><<<blocks, 256, 0, s>>>(df_rows, by_point, by_point_bounds, \
                                                                     by_point_starts, g.n, g.c_in, d_feats)
        if (lanes == 8) ROWS_GO(8);
        else if (lanes == 16) ROWS_GO(16);
        else if (lanes == 32) ROWS_GO(32);
        else ROWS_GO(64);
#undef ROWS_GO
        PCCNN_LAUNCH_CHECK();
    }
    if (gather) {
        conv_point_gather_kernel<<<(unsigned)pccnn_ceil_div(g.n * 4, 256), 256, 0, s>>>(
            pair_grads, by_point, by_point_bounds, by_point_starts, g.n, o.d_pts, o.d_pdf);
        PCCNN_LAUNCH_CHECK();
    }
    if (o.partials) {
        if (det) conv_param_reduce1_compact_kernel<<<reduce_groups, 256, 0, s>>>(partials, partial_rows, kpad_of(g.k), stage);
        else conv_param_reduce1_kernel<<<reduce_groups, 256, 0, s>>>(partials, partial_rows, stage);
        PCCNN_LAUNCH_CHECK();
        conv_param_reduce2_kernel<BASIS><<<1, 256, 0, s>>>(stage, reduce_groups, g.k, d_param_a, d_param_b);
        PCCNN_LAUNCH_CHECK();
    }
    return PCCNN_OK;
}

template <int BASIS>
static int conv_weight_var(ConvGeom g, const float *feats, float *out, void *workspace, size_t workspace_bytes,
                           hipStream_t s, bool divide_by_count = false)
{
    PCCNN_REQUIRE(g.m > 0, PCCNN_ERR_INVALID, "conv weight variance: no samples");
    PccnnArena arena(workspace, workspace_bytes);
    float *proj = arena.take<float>((size_t)g.m * g.c_in * g.k);
    float *rows = arena.take<float>((size_t)g.m);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv weight variance: workspace of %zu bytes, need %zu",
                  workspace_bytes, pccnn_conv_weight_var_workspace_bytes(g.m, 0, g.c_in, g.k));
    int rc = launch_proj_fwd<BASIS>(g, feats, proj, s);
    if (rc != PCCNN_OK) return rc;
    row_sumsq_kernel<<<(unsigned)pccnn_ceil_div(g.m, 4), 256, 0, s>>>(proj, g.m, (int64_t)g.c_in * g.k, rows);
    PCCNN_LAUNCH_CHECK();
    if (divide_by_count) {
        divide_by_count_sq_kernel<<<(unsigned)pccnn_ceil_div(g.m, 256), 256, 0, s>>>(rows, g.ends, g.m);
        PCCNN_LAUNCH_CHECK();
    }
    mean_reciprocal_kernel<<<1, 256, 0, s>>>(rows, g.m, out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// Defined with the generic entry points below; the dedicated entry points hand clouds that are not 3-D to them.
static int conv_forward_entry(const char *who, bool bf16, const pccnn_basis *basis, const float *pts, const float *feats,
                              const float *samples, const int32_t *neigh, const int32_t *ends, const float *radii,
                              const float *weights, int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps,
                              int c_out, int divide_by_count, float *out, void *proj_out, void *workspace,
                              size_t workspace_bytes, void *stream);
static int conv_backward_entry(const char *who, bool bf16, const pccnn_basis *basis, const float *pts, const float *feats,
                                   const float *samples, const int32_t *neigh, const int32_t *ends,
                                   const float *radii, const float *weights, const float *in_grads, const void *proj,
                                   const int32_t *mirror, int grad_mask, int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps,
                                   int c_out, int divide_by_count, float *d_weights, float *d_feats, float *d_param_a,
                                   float *d_param_b, float *d_pdf, float *d_pts, float *d_samples, void *workspace,
                                   size_t workspace_bytes, void *stream);

extern "C" size_t pccnn_conv_weight_var_workspace_bytes(int64_t m, int64_t t, int c_in, int k)
{
    if (m < 1) m = 1;
    if (t < 1) t = 1;
    // projection, per-sample sums and (for clouds that are not 3-D) the per-pair basis
    return pccnn_align((size_t)m * c_in * k * sizeof(float)) + pccnn_align((size_t)m * sizeof(float)) +
           pccnn_align((size_t)t * k * sizeof(float)) + 256;
}

extern "C" int pccnn_kpconv_weight_var(const float *pts, const float *feats, const float *samples,
                                       const int32_t *neigh, const int32_t *ends, const float *radii,
                                       const float *kernel_pts, float sigma, int64_t n, int64_t m, int64_t t, int d,
                                       int c_in, int k, float *out, void *workspace, size_t workspace_bytes,
                                       void *stream)
{
    if (d != 3) {
        const pccnn_basis b = {PCCNN_BASIS_KP, k, kernel_pts, nullptr, nullptr, 0, 0, 0, sigma, nullptr};
        return pccnn_conv_weight_var(&b, pts, feats, samples, neigh, ends, radii, n, m, t, d, c_in, 0, out, workspace,
                                     workspace_bytes, stream);
    }
    int rc = conv_validate("pccnn_kpconv_weight_var", n, m, t, d, c_in, k, 1, 1);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(sigma > 0.0f, PCCNN_ERR_INVALID, "pccnn_kpconv_weight_var: sigma=%g", sigma);
    PCCNN_REQUIRE(pts && feats && samples && ends && radii && kernel_pts && out && (t == 0 || neigh), PCCNN_ERR_INVALID,
                  "pccnn_kpconv_weight_var: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, nullptr, kernel_pts, nullptr, sigma, n, m, t, c_in, k};
    return conv_weight_var<BASIS_KP>(g, feats, out, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int pccnn_mcconv_weight_var(const float *pts, const float *pdf, const float *feats, const float *samples,
                                       const int32_t *neigh, const int32_t *ends, const float *radii,
                                       const float *axis, const float *bias, int64_t n, int64_t m, int64_t t, int d,
                                       int c_in, int k, float *out, void *workspace, size_t workspace_bytes,
                                       void *stream)
{
    if (d != 3) {
        const pccnn_basis b = {PCCNN_BASIS_MLP, k, axis, bias, nullptr, 0, 0, 0, 1.0f, pdf};
        return pccnn_conv_weight_var(&b, pts, feats, samples, neigh, ends, radii, n, m, t, d, c_in, 0, out, workspace,
                                     workspace_bytes, stream);
    }
    int rc = conv_validate("pccnn_mcconv_weight_var", n, m, t, d, c_in, k, 1, 1);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(pts && pdf && feats && samples && ends && radii && axis && bias && out && (t == 0 || neigh),
                  PCCNN_ERR_INVALID, "pccnn_mcconv_weight_var: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, pdf, axis, bias, 1.0f, n, m, t, c_in, k};
    return conv_weight_var<BASIS_MLP>(g, feats, out, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int pccnn_kpconv_forward(const float *pts, const float *feats, const float *samples, const int32_t *neigh,
                                    const int32_t *ends, const float *radii, const float *kernel_pts, float sigma,
                                    const float *weights, int64_t n, int64_t m, int64_t t, int d, int c_in, int k,
                                    int c_out, float *out, float *proj_out, void *workspace, size_t workspace_bytes,
                                    void *stream)
{
    if (d != 3) {
        const pccnn_basis b = {PCCNN_BASIS_KP, k, kernel_pts, nullptr, nullptr, 0, 0, 0, sigma, nullptr};
        return conv_forward_entry("pccnn_kpconv_forward", false, &b, pts, feats, samples, neigh, ends, radii, weights, n,
                                  m, t, d, c_in, 1, c_out, 0, out, proj_out, workspace, workspace_bytes, stream);
    }
    int rc = conv_validate("pccnn_kpconv_forward", n, m, t, d, c_in, k, 1, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(sigma > 0.0f, PCCNN_ERR_INVALID, "pccnn_kpconv_forward: sigma=%g", sigma);
    PCCNN_REQUIRE(m == 0 || (pts && feats && samples && ends && radii && kernel_pts && weights && out && (t == 0 || neigh)),
                  PCCNN_ERR_INVALID, "pccnn_kpconv_forward: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, nullptr, kernel_pts, nullptr, sigma, n, m, t, c_in, k};
    return conv_forward<BASIS_KP>(g, feats, weights, 1, c_out, out, proj_out, workspace, workspace_bytes,
                                  (hipStream_t)stream);
}

extern "C" int pccnn_kpconv_backward(const float *pts, const float *feats, const float *samples,
                                     const int32_t *neigh, const int32_t *ends, const float *radii,
                                     const float *kernel_pts, float sigma, const float *weights,
                                     const float *in_grads, const float *proj, const int32_t *mirror, int grad_mask,
                                     int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int c_out,
                                     float *d_weights, float *d_feats, float *d_kernel_pts, float *d_pts,
                                     float *d_samples, void *workspace, size_t workspace_bytes, void *stream)
{
    if (d != 3) {
        const pccnn_basis b = {PCCNN_BASIS_KP, k, kernel_pts, nullptr, nullptr, 0, 0, 0, sigma, nullptr};
        return conv_backward_entry("pccnn_kpconv_backward", false, &b, pts, feats, samples, neigh, ends, radii, weights,
                                   in_grads, proj, mirror, grad_mask, n, m, t, d, c_in, 1, c_out, 0, d_weights, d_feats,
                                   d_kernel_pts, nullptr, nullptr, d_pts, d_samples, workspace, workspace_bytes, stream);
    }
    int rc = conv_validate("pccnn_kpconv_backward", n, m, t, d, c_in, k, 1, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(mirror == nullptr || n == m, PCCNN_ERR_INVALID,
                  "pccnn_kpconv_backward: a mirror index needs samples == points (n=%lld, m=%lld)", (long long)n,
                  (long long)m);
    PCCNN_REQUIRE(sigma > 0.0f, PCCNN_ERR_INVALID, "pccnn_kpconv_backward: sigma=%g", sigma);
    PCCNN_REQUIRE(kernel_pts && weights && radii && (n == 0 || (pts && feats)) &&
                      (m == 0 || (samples && ends && in_grads)) && (t == 0 || neigh),
                  PCCNN_ERR_INVALID, "pccnn_kpconv_backward: null input pointer");
    PCCNN_REQUIRE((!(grad_mask & PCCNN_GRAD_WEIGHTS) || d_weights) && (!(grad_mask & PCCNN_GRAD_FEATS) || d_feats || n == 0) &&
                      (!(grad_mask & PCCNN_GRAD_BASIS_PARAMS) || d_kernel_pts) &&
                      (!(grad_mask & PCCNN_GRAD_PTS) || ((d_pts || n == 0) && (d_samples || m == 0))),
                  PCCNN_ERR_INVALID, "pccnn_kpconv_backward: a requested gradient has a null output pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, nullptr, kernel_pts, nullptr, sigma, n, m, t, c_in, k};
    return conv_backward<BASIS_KP>(g, feats, weights, in_grads, 1, c_out, proj, grad_mask, d_weights, d_feats,
                                   d_kernel_pts, nullptr, nullptr, d_pts, d_samples, workspace, workspace_bytes,
                                   (hipStream_t)stream, false, mirror);
}

extern "C" int pccnn_mcconv_forward(const float *pts, const float *pdf, const float *feats, const float *samples,
                                    const int32_t *neigh, const int32_t *ends, const float *radii, const float *axis,
                                    const float *bias, const float *weights, int64_t n, int64_t m, int64_t t, int d,
                                    int c_in, int k, int num_mlps, int c_out, float *out, float *proj_out,
                                    void *workspace, size_t workspace_bytes, void *stream)
{
    if (d != 3) {
        const pccnn_basis b = {PCCNN_BASIS_MLP, k, axis, bias, nullptr, 0, 0, 0, 1.0f, pdf};
        return conv_forward_entry("pccnn_mcconv_forward", false, &b, pts, feats, samples, neigh, ends, radii, weights, n,
                                  m, t, d, c_in, num_mlps, c_out, 0, out, proj_out, workspace, workspace_bytes, stream);
    }
    int rc = conv_validate("pccnn_mcconv_forward", n, m, t, d, c_in, k, num_mlps, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(m == 0 || (pts && pdf && feats && samples && ends && radii && axis && bias && weights && out &&
                             (t == 0 || neigh)),
                  PCCNN_ERR_INVALID, "pccnn_mcconv_forward: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, pdf, axis, bias, 1.0f, n, m, t, c_in, k};
    return conv_forward<BASIS_MLP>(g, feats, weights, num_mlps, c_out, out, proj_out, workspace, workspace_bytes,
                                   (hipStream_t)stream);
}

extern "C" int pccnn_mcconv_backward(const float *pts, const float *pdf, const float *feats, const float *samples,
                                     const int32_t *neigh, const int32_t *ends, const float *radii,
                                     const float *axis, const float *bias, const float *weights,
                                     const float *in_grads, const float *proj, const int32_t *mirror, int grad_mask,
                                     int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int num_mlps, int c_out,
                                     float *d_weights, float *d_feats, float *d_axis, float *d_bias, float *d_pdf,
                                     float *d_pts, float *d_samples, void *workspace, size_t workspace_bytes,
                                     void *stream)
{
    if (d != 3) {
        const pccnn_basis b = {PCCNN_BASIS_MLP, k, axis, bias, nullptr, 0, 0, 0, 1.0f, pdf};
        return conv_backward_entry("pccnn_mcconv_backward", false, &b, pts, feats, samples, neigh, ends, radii, weights,
                                   in_grads, proj, mirror, grad_mask, n, m, t, d, c_in, num_mlps, c_out, 0, d_weights,
                                   d_feats, d_axis, d_bias, d_pdf, d_pts, d_samples, workspace, workspace_bytes, stream);
    }
    int rc = conv_validate("pccnn_mcconv_backward", n, m, t, d, c_in, k, num_mlps, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(mirror == nullptr || n == m, PCCNN_ERR_INVALID,
                  "pccnn_mcconv_backward: a mirror index needs samples == points (n=%lld, m=%lld)", (long long)n,
                  (long long)m);
    PCCNN_REQUIRE(axis && bias && weights && radii && (n == 0 || (pts && pdf && feats)) &&
                      (m == 0 || (samples && ends && in_grads)) && (t == 0 || neigh),
                  PCCNN_ERR_INVALID, "pccnn_mcconv_backward: null input pointer");
    PCCNN_REQUIRE((!(grad_mask & PCCNN_GRAD_WEIGHTS) || d_weights) && (!(grad_mask & PCCNN_GRAD_FEATS) || d_feats || n == 0) &&
                      (!(grad_mask & PCCNN_GRAD_BASIS_PARAMS) || (d_axis && d_bias)) &&
                      (!(grad_mask & PCCNN_GRAD_PDF) || d_pdf || n == 0) &&
                      (!(grad_mask & PCCNN_GRAD_PTS) || ((d_pts || n == 0) && (d_samples || m == 0))),
                  PCCNN_ERR_INVALID, "pccnn_mcconv_backward: a requested gradient has a null output pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, pdf, axis, bias, 1.0f, n, m, t, c_in, k};
    return conv_backward<BASIS_MLP>(g, feats, weights, in_grads, num_mlps, c_out, proj, grad_mask, d_weights, d_feats,
                                    d_axis, d_bias, d_pdf, d_pts, d_samples, workspace, workspace_bytes,
                                    (hipStream_t)stream, false, mirror);
}

// ---------------------------------------------------------------- other dimensions (2, 4, 5, 6)
// The fused kernels above are written for three dimensions.  In any other dimension the basis is evaluated per
// pair into a [T, K] tensor by the kernel below, the convolution then runs with that tensor as a caller-given basis
// (the EXPLICIT family: projection, contraction, projection backward unchanged), and a second per-pair kernel turns
// the basis gradient it returns into the point, sample, density and basis-parameter gradients.  Same formulas as
// LaneBasis::eval and basis_derivative, with the sums over the dimensions in order from 0.

struct PairGeom {
    const float *pts, *samples;     // [n,d], [m,d]
    const int2 *neigh;              // [t] (point, sample)
    const float *radii;             // [d]
    const float *pdf;               // [n] or null
    const float *a, *b;             // kernel points [k,d] | axis [d,k]; bias [k]
    float sigma;
    int64_t t;
    int d, k;
};

template <int BASIS>
__global__ void __launch_bounds__(256)
pair_basis_fwd_kernel(PairGeom g, float *__restrict__ basis)
{
#pragma clang fp contract(off)
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= g.t * g.k) return;
    const int64_t t = idx / g.k;
    const int k = (int)(idx - t * g.k);
    const int2 pr = g.neigh[t];
    float acc = 0.0f;
    for (int i = 0; i < g.d; ++i) {
        const float diff = (g.pts[(int64_t)pr.x * g.d + i] - g.samples[(int64_t)pr.y * g.d + i]) * (1.0f / g.radii[i]);
        if (BasisTraits<BASIS>::kernel_pts) {
            const float v = g.a[k * g.d + i] - diff;
            acc = acc + v * v;
        } else {
            acc = acc + diff * g.a[i * g.k + k];
        }
    }
    float w;
    if (BASIS == BASIS_KP || BASIS == BASIS_KPN) {
        const float r = 1.0f - sqrtf(fmaxf(acc, 0.0f)) / g.sigma;
        w = fminf(fmaxf(r, 0.0f), 1.0f);
        if (BASIS == BASIS_KPN) w = w / g.pdf[pr.x];
    } else if (BASIS == BASIS_GAUSS) {
        w = expf(-(acc / (2.0f * g.sigma * g.sigma))) / g.pdf[pr.x];
    } else if (BASIS == BASIS_LINEAR) {
        w = acc + g.b[k];
    } else {
        acc = acc + g.b[k];
        acc = acc > 0.0f ? acc : acc * 0.2f;
        w = acc / g.pdf[pr.x];
    }
    basis[idx] = w;
}

// One thread per pair, a loop over the basis index.  Parameter gradients are summed per workgroup in LDS
// ([k][d + 1]) and flushed with one float atomic per entry; the point-side gradients are float atomics per pair.
template <int BASIS>
__global__ void __launch_bounds__(256)
pair_basis_bwd_kernel(PairGeom g, const float *__restrict__ basis_grads, float *d_pts, float *d_samples,
                      float *d_pdf, float *d_a, float *d_b)
{
#pragma clang fp contract(off)
    __shared__ float part[64 * (PCCNN_MAX_DIMS + 1)];
    const int comps = g.d + 1;
    for (int i = threadIdx.x; i < g.k * comps; i += blockDim.x) part[i] = 0.0f;
    __syncthreads();
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < g.t) {
        const int2 pr = g.neigh[t];
        float diff[PCCNN_MAX_DIMS], ir[PCCNN_MAX_DIMS], gd[PCCNN_MAX_DIMS];
        for (int i = 0; i < PCCNN_MAX_DIMS; ++i) {
            diff[i] = 0.0f; ir[i] = 0.0f; gd[i] = 0.0f;
            if (i < g.d) {
                ir[i] = 1.0f / g.radii[i];
                diff[i] = (g.pts[(int64_t)pr.x * g.d + i] - g.samples[(int64_t)pr.y * g.d + i]) * ir[i];
            }
        }
        const float pdf = BasisTraits<BASIS>::uses_pdf ? g.pdf[pr.x] : 1.0f;
        float gpdf = 0.0f;
        for (int k = 0; k < g.k; ++k) {
            const float gk = basis_grads[t * g.k + k];
            if (BasisTraits<BASIS>::kernel_pts) {
                float v[PCCNN_MAX_DIMS];
                float acc = 0.0f;
                for (int i = 0; i < PCCNN_MAX_DIMS; ++i) {
                    v[i] = 0.0f;
                    if (i < g.d) { v[i] = g.a[k * g.d + i] - diff[i]; acc = acc + v[i] * v[i]; }
                }
                float c = 0.0f;
                if (BASIS == BASIS_GAUSS) {
                    const float e = expf(-(acc / (2.0f * g.sigma * g.sigma)));
                    gpdf += -((e / pdf) * gk) / pdf;
                    c = -(gk / pdf) * e * (1.0f / (g.sigma * g.sigma));
                } else {
                    const float gin = (BASIS == BASIS_KPN) ? gk / pdf : gk;
                    const float dist = sqrtf(fmaxf(acc, 0.0f));
                    if (1.0f - dist / g.sigma >= 0.0f) c = -(gin / g.sigma) * (1.0f / (dist + 1e-6f));
                }
                for (int i = 0; i < PCCNN_MAX_DIMS; ++i)
                    if (i < g.d) {
                        const float ci = c * v[i];
                        gd[i] -= ci;
                        if (d_a && ci != 0.0f) atomicAdd(&part[k * comps + i], ci);
                    }
            } else {
                float act = 0.0f;
                for (int i = 0; i < PCCNN_MAX_DIMS; ++i)
                    if (i < g.d) act = act + diff[i] * g.a[i * g.k + k];
                act = act + g.b[k];
                const bool pos = act > 0.0f || BASIS == BASIS_LINEAR;
                act = pos ? act : act * 0.2f;
                const float inv_pd = 1.0f / pdf;
                gpdf += -(act * gk * inv_pd * inv_pd);
                const float c = gk * inv_pd * (pos ? 1.0f : 0.2f);
                for (int i = 0; i < PCCNN_MAX_DIMS; ++i)
                    if (i < g.d) {
                        gd[i] += c * g.a[i * g.k + k];
                        if (d_a) atomicAdd(&part[k * comps + i], diff[i] * c);
                    }
                if (d_b) atomicAdd(&part[k * comps + g.d], c);
            }
        }
        for (int i = 0; i < PCCNN_MAX_DIMS; ++i)
            if (i < g.d) {
                const float v = gd[i] * ir[i];
                if (d_pts) unsafeAtomicAdd(&d_pts[(int64_t)pr.x * g.d + i], v);
                if (d_samples) unsafeAtomicAdd(&d_samples[(int64_t)pr.y * g.d + i], -v);
            }
        if (BasisTraits<BASIS>::pdf_grad && d_pdf) unsafeAtomicAdd(&d_pdf[pr.x], gpdf);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < g.k * comps; i += blockDim.x) {
        const int k = i / comps, c = i - k * comps;
        const float v = part[i];
        if (v == 0.0f) continue;
        if (c < g.d) {
            // kernel points are stored [k][d], axis matrices [d][k]
            if (d_a) unsafeAtomicAdd(&d_a[BasisTraits<BASIS>::kernel_pts ? k * g.d + c : c * g.k + k], v);
        } else if (d_b) {
            unsafeAtomicAdd(&d_b[k], v);
        }
    }
}

#define PAIR_BASIS_LINEAR (-1)   // PointConv's affine basis; not one of the public PCCNN_BASIS_* kinds

static bool pair_basis_kind(int kind)
{
    return kind == PCCNN_BASIS_KP || kind == PCCNN_BASIS_MLP || kind == PCCNN_BASIS_KPN || kind == PCCNN_BASIS_GAUSS;
}

static int pair_basis_forward(int kind, const PairGeom &g, float *basis, hipStream_t s)
{
    if (g.t == 0) return PCCNN_OK;
    const unsigned blocks = (unsigned)pccnn_ceil_div(g.t * g.k, 256);
    switch (kind) {
    case PCCNN_BASIS_KP: pair_basis_fwd_kernel<BASIS_KP><<<blocks, 256, 0, s>>>(g, basis); break;
    case PCCNN_BASIS_MLP: pair_basis_fwd_kernel<BASIS_MLP><<<blocks, 256, 0, s>>>(g, basis); break;
    case PCCNN_BASIS_KPN: pair_basis_fwd_kernel<BASIS_KPN><<<blocks, 256, 0, s>>>(g, basis); break;
    case PAIR_BASIS_LINEAR: pair_basis_fwd_kernel<BASIS_LINEAR><<<blocks, 256, 0, s>>>(g, basis); break;
    default: pair_basis_fwd_kernel<BASIS_GAUSS><<<blocks, 256, 0, s>>>(g, basis); break;
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

static int pair_basis_backward(int kind, const PairGeom &g, const float *basis_grads, float *d_pts, float *d_samples,
                               float *d_pdf, float *d_a, float *d_b, hipStream_t s)
{
    if (g.t == 0) return PCCNN_OK;
    const unsigned blocks = (unsigned)pccnn_ceil_div(g.t, 256);
    switch (kind) {
    case PCCNN_BASIS_KP:
        pair_basis_bwd_kernel<BASIS_KP><<<blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, d_pdf, d_a, d_b); break;
    case PCCNN_BASIS_MLP:
        pair_basis_bwd_kernel<BASIS_MLP><<<blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, d_pdf, d_a, d_b); break;
    case PCCNN_BASIS_KPN:
        pair_basis_bwd_kernel<BASIS_KPN><<<blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, d_pdf, d_a, d_b); break;
    case PAIR_BASIS_LINEAR:
        pair_basis_bwd_kernel<BASIS_LINEAR><<<blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, d_pdf, d_a, d_b); break;
    default:
        pair_basis_bwd_kernel<BASIS_GAUSS><<<blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, d_pdf, d_a, d_b); break;
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// The part of a workspace that is left after `bytes` have been set aside at its start.
static void *ws_after(void *workspace, size_t workspace_bytes, size_t bytes, size_t &rest)
{
    bytes = pccnn_align(bytes);
    if (workspace == nullptr || workspace_bytes < bytes) { rest = 0; return nullptr; }
    rest = workspace_bytes - bytes;
    return (char *)workspace + bytes;
}

// ------------------------------------------------------------------- generic entry points

static int basis_geom(const char *who, const pccnn_basis *b, const float *pts, const float *samples,
                      const int32_t *neigh, const int32_t *ends, const float *radii, int64_t n, int64_t m, int64_t t,
                      int c_in, ConvGeom &g)
{
    PCCNN_REQUIRE(b != nullptr, PCCNN_ERR_INVALID, "%s: null basis descriptor", who);
    PCCNN_REQUIRE(b->kind >= PCCNN_BASIS_KP && b->kind <= PCCNN_BASIS_SPH, PCCNN_ERR_INVALID, "%s: basis kind %d", who,
                  b->kind);
    int k = b->k;
    if (b->kind == PCCNN_BASIS_SPH) {
        PCCNN_REQUIRE(b->nb0 > 0 && b->nb1 > 0 && b->nb2 > 0 && b->a && b->b && b->c, PCCNN_ERR_INVALID,
                      "%s: spherical basis needs three non-empty bin edge arrays", who);
        k = b->nb0 * b->nb1 * b->nb2 + 1;
    } else {
        PCCNN_REQUIRE(b->a != nullptr || (b->kind == PCCNN_BASIS_EXPLICIT && t == 0), PCCNN_ERR_INVALID,
                      "%s: null basis parameter", who);
    }
    PCCNN_REQUIRE(k >= 1 && k <= 64, PCCNN_ERR_UNSUPPORTED, "%s: basis size k=%d outside [1,64]", who, k);
    const bool kp = b->kind == PCCNN_BASIS_KP || b->kind == PCCNN_BASIS_KPN || b->kind == PCCNN_BASIS_GAUSS;
    const bool with_pdf = b->kind == PCCNN_BASIS_MLP || b->kind == PCCNN_BASIS_KPN || b->kind == PCCNN_BASIS_GAUSS;
    PCCNN_REQUIRE(!kp || b->sigma > 0.0f, PCCNN_ERR_INVALID, "%s: sigma=%g", who, b->sigma);
    PCCNN_REQUIRE(!with_pdf || b->pdf || n == 0, PCCNN_ERR_INVALID, "%s: this basis needs the point densities", who);
    PCCNN_REQUIRE(b->kind != PCCNN_BASIS_MLP || b->b, PCCNN_ERR_INVALID, "%s: null bias", who);
    g = ConvGeom{pts, samples, (const int2 *)neigh, ends, radii, b->pdf, b->a, b->b, b->sigma, n, m, t, c_in, k,
                 b->c, b->nb0, b->nb1, b->nb2};
    return PCCNN_OK;
}

#define BASIS_DISPATCH(kind, CALL)                                                       \
    switch (kind) {                                                                      \
    case PCCNN_BASIS_KP: return CALL(BASIS_KP);                                          \
    case PCCNN_BASIS_MLP: return CALL(BASIS_MLP);                                        \
    case PCCNN_BASIS_KPN: return CALL(BASIS_KPN);                                        \
    case PCCNN_BASIS_GAUSS: return CALL(BASIS_GAUSS);                                    \
    case PCCNN_BASIS_EXPLICIT: return CALL(BASIS_EXPLICIT);                              \
    default: return CALL(BASIS_SPH);                                                     \
    }

static int conv_forward_entry(const char *who, bool bf16, const pccnn_basis *basis, const float *pts, const float *feats,
                                  const float *samples, const int32_t *neigh, const int32_t *ends, const float *radii,
                                  const float *weights, int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps,
                                  int c_out, int divide_by_count, float *out, void *proj_out, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    ConvGeom g;
    int rc = basis_geom(who, basis, pts, samples, neigh, ends, radii, n, m, t, c_in, g);
    if (rc != PCCNN_OK) return rc;
    if ((rc = conv_validate(who, n, m, t, d, c_in, g.k, num_mlps, c_out)) != PCCNN_OK) return rc;
    const bool geom = basis->kind != PCCNN_BASIS_EXPLICIT;
    PCCNN_REQUIRE(m == 0 || (feats && ends && weights && out && (t == 0 || neigh) && (!geom || (pts && samples && radii))),
                  PCCNN_ERR_INVALID, "%s: null pointer", who);
    if (d != 3 && geom) {
        // basis per pair, then the convolution on it as a caller-given basis
        PCCNN_REQUIRE(pair_basis_kind(basis->kind), PCCNN_ERR_UNSUPPORTED, "%s: basis kind %d needs 3 dimensions (d=%d)",
                      who, basis->kind, d);
        if (m == 0) return PCCNN_OK;
        size_t rest = 0;
        void *ws = ws_after(workspace, workspace_bytes, (size_t)(t > 0 ? t : 1) * g.k * sizeof(float), rest);
        PCCNN_REQUIRE(ws != nullptr, PCCNN_ERR_WORKSPACE, "%s: workspace of %zu bytes, need %zu", who, workspace_bytes,
                      pccnn_conv_workspace_bytes(m, t, c_in, g.k, c_out, 0));
        float *pair_w = (float *)workspace;
        const PairGeom pg = {pts, samples, (const int2 *)neigh, radii, basis->pdf, basis->a, basis->b, basis->sigma, t, d,
                             g.k};
        if ((rc = pair_basis_forward(basis->kind, pg, pair_w, (hipStream_t)stream)) != PCCNN_OK) return rc;
        ConvGeom ge = {nullptr, nullptr, (const int2 *)neigh, ends, nullptr, nullptr, pair_w, nullptr, 1.0f, n, m, t,
                       c_in, g.k};
        return conv_forward<BASIS_EXPLICIT>(ge, feats, weights, num_mlps, c_out, out, proj_out, ws, rest,
                                            (hipStream_t)stream, divide_by_count != 0, bf16);
    }
#define CALL(B) conv_forward<B>(g, feats, weights, num_mlps, c_out, out, proj_out, workspace, workspace_bytes, \
                                (hipStream_t)stream, divide_by_count != 0, bf16)
    BASIS_DISPATCH(basis->kind, CALL)
#undef CALL
}

extern "C" int pccnn_conv_forward(const pccnn_basis *basis, const float *pts, const float *feats,
                                  const float *samples, const int32_t *neigh, const int32_t *ends, const float *radii,
                                  const float *weights, int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps,
                                  int c_out, int divide_by_count, float *out, float *proj_out, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    return conv_forward_entry("pccnn_conv_forward", false, basis, pts, feats, samples, neigh, ends, radii, weights, n, m,
                              t, d, c_in, num_mlps, c_out, divide_by_count, out, proj_out, workspace, workspace_bytes,
                              stream);
}

extern "C" int pccnn_conv_forward_bf16(const pccnn_basis *basis, const float *pts, const float *feats,
                                       const float *samples, const int32_t *neigh, const int32_t *ends,
                                       const float *radii, const float *weights, int64_t n, int64_t m, int64_t t, int d,
                                       int c_in, int num_mlps, int c_out, int divide_by_count, float *out,
                                       uint16_t *proj_out, void *workspace, size_t workspace_bytes, void *stream)
{
    return conv_forward_entry("pccnn_conv_forward_bf16", true, basis, pts, feats, samples, neigh, ends, radii, weights,
                              n, m, t, d, c_in, num_mlps, c_out, divide_by_count, out, proj_out, workspace,
                              workspace_bytes, stream);
}

static int conv_backward_entry(const char *who, bool bf16, const pccnn_basis *basis, const float *pts, const float *feats,
                                   const float *samples, const int32_t *neigh, const int32_t *ends,
                                   const float *radii, const float *weights, const float *in_grads, const void *proj,
                                   const int32_t *mirror, int grad_mask, int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps,
                                   int c_out, int divide_by_count, float *d_weights, float *d_feats, float *d_param_a,
                                   float *d_param_b, float *d_pdf, float *d_pts, float *d_samples, void *workspace,
                                   size_t workspace_bytes, void *stream)
{
    ConvGeom g;
    int rc = basis_geom(who, basis, pts, samples, neigh, ends, radii, n, m, t, c_in, g);
    if (rc != PCCNN_OK) return rc;
    if ((rc = conv_validate(who, n, m, t, d, c_in, g.k, num_mlps, c_out)) != PCCNN_OK) return rc;
    PCCNN_REQUIRE(mirror == nullptr || n == m, PCCNN_ERR_INVALID,
                  "%s: a mirror index needs samples == points (n=%lld, m=%lld)", who, (long long)n,
                  (long long)m);
    const int kind = basis->kind;
    const bool geom = kind != PCCNN_BASIS_EXPLICIT;
    PCCNN_REQUIRE(weights && (n == 0 || feats) && (m == 0 || (ends && in_grads)) && (t == 0 || neigh) &&
                      (!geom || (radii && (n == 0 || pts) && (m == 0 || samples))),
                  PCCNN_ERR_INVALID, "%s: null input pointer", who);
    const bool has_param = kind != PCCNN_BASIS_SPH;
    const bool has_pts = kind != PCCNN_BASIS_SPH && kind != PCCNN_BASIS_EXPLICIT;
    const bool has_pdf = kind == PCCNN_BASIS_MLP || kind == PCCNN_BASIS_GAUSS;
    PCCNN_REQUIRE((!(grad_mask & PCCNN_GRAD_WEIGHTS) || d_weights) &&
                      (!(grad_mask & PCCNN_GRAD_FEATS) || d_feats || n == 0) &&
                      (!(grad_mask & PCCNN_GRAD_BASIS_PARAMS) || !has_param || d_param_a) &&
                      (!(grad_mask & PCCNN_GRAD_BASIS_PARAMS) || kind != PCCNN_BASIS_MLP || d_param_b) &&
                      (!(grad_mask & PCCNN_GRAD_PDF) || !has_pdf || d_pdf || n == 0) &&
                      (!(grad_mask & PCCNN_GRAD_PTS) || !has_pts || ((d_pts || n == 0) && (d_samples || m == 0))),
                  PCCNN_ERR_INVALID, "%s: a requested gradient has a null output pointer", who);
    if (d != 3 && geom) {
        PCCNN_REQUIRE(pair_basis_kind(kind), PCCNN_ERR_UNSUPPORTED, "%s: basis kind %d needs 3 dimensions (d=%d)", who,
                      kind, d);
        PCCNN_REQUIRE(!(grad_mask & PCCNN_GRAD_DETERMINISTIC), PCCNN_ERR_UNSUPPORTED,
                      "%s: the pass without atomics (PCCNN_GRAD_DETERMINISTIC) is three-dimensional, d=%d", who, d);
        hipStream_t s = (hipStream_t)stream;
        const bool want_par = grad_mask & PCCNN_GRAD_BASIS_PARAMS, want_pts = grad_mask & PCCNN_GRAD_PTS;
        const bool want_pdf = (grad_mask & PCCNN_GRAD_PDF) && has_pdf;
        const bool want_basis = want_par || want_pts || want_pdf;
        // outputs of the per-pair stage are accumulated with atomics: they start at zero
        if (want_pts && (rc = pccnn_fill_f32(d_pts, 0.0f, n * d, s)) != PCCNN_OK) return rc;
        if (want_pts && (rc = pccnn_fill_f32(d_samples, 0.0f, m * d, s)) != PCCNN_OK) return rc;
        if (want_pdf && (rc = pccnn_fill_f32(d_pdf, 0.0f, n, s)) != PCCNN_OK) return rc;
        if (want_par && (rc = pccnn_fill_f32(d_param_a, 0.0f, (int64_t)g.k * d, s)) != PCCNN_OK) return rc;
        if (want_par && kind == PCCNN_BASIS_MLP && (rc = pccnn_fill_f32(d_param_b, 0.0f, g.k, s)) != PCCNN_OK) return rc;
        const size_t tk = (size_t)(t > 0 ? t : 1) * g.k * sizeof(float);
        size_t rest = 0;
        void *ws = ws_after(workspace, workspace_bytes, 2 * pccnn_align(tk), rest);
        PCCNN_REQUIRE(ws != nullptr, PCCNN_ERR_WORKSPACE, "%s: workspace of %zu bytes, need %zu", who, workspace_bytes,
                      pccnn_conv_workspace_bytes(m, t, c_in, g.k, c_out, 1));
        float *pair_w = (float *)workspace;
        float *pair_g = (float *)((char *)workspace + pccnn_align(tk));
        const PairGeom pg = {pts, samples, (const int2 *)neigh, radii, basis->pdf, basis->a, basis->b, basis->sigma, t, d,
                             g.k};
        if (m > 0 && (rc = pair_basis_forward(kind, pg, pair_w, s)) != PCCNN_OK) return rc;
        ConvGeom ge = {nullptr, nullptr, (const int2 *)neigh, ends, nullptr, nullptr, pair_w, nullptr, 1.0f, n, m, t,
                       c_in, g.k};
        const int mask = (grad_mask & (PCCNN_GRAD_WEIGHTS | PCCNN_GRAD_FEATS)) | (want_basis ? PCCNN_GRAD_BASIS_PARAMS : 0);
        rc = conv_backward<BASIS_EXPLICIT>(ge, feats, weights, in_grads, num_mlps, c_out, proj, mask, d_weights, d_feats,
                                           pair_g, nullptr, nullptr, nullptr, nullptr, ws, rest, s, divide_by_count != 0,
                                           nullptr, bf16);
        if (rc != PCCNN_OK || !want_basis || m == 0 || t == 0) return rc;
        return pair_basis_backward(kind, pg, pair_g, want_pts ? d_pts : nullptr, want_pts ? d_samples : nullptr,
                                   want_pdf ? d_pdf : nullptr, want_par ? d_param_a : nullptr,
                                   want_par ? d_param_b : nullptr, s);
    }
#define CALL(B) conv_backward<B>(g, feats, weights, in_grads, num_mlps, c_out, proj, grad_mask, d_weights, d_feats, \
                                 d_param_a, d_param_b, d_pdf, d_pts, d_samples, workspace, workspace_bytes,           \
                                 (hipStream_t)stream, divide_by_count != 0, mirror, bf16)
    BASIS_DISPATCH(kind, CALL)
#undef CALL
}

extern "C" int pccnn_conv_backward(const pccnn_basis *basis, const float *pts, const float *feats,
                                   const float *samples, const int32_t *neigh, const int32_t *ends,
                                   const float *radii, const float *weights, const float *in_grads, const float *proj,
                                   const int32_t *mirror, int grad_mask, int64_t n, int64_t m, int64_t t, int d, int c_in,
                                   int num_mlps, int c_out, int divide_by_count, float *d_weights, float *d_feats,
                                   float *d_param_a, float *d_param_b, float *d_pdf, float *d_pts, float *d_samples,
                                   void *workspace, size_t workspace_bytes, void *stream)
{
    return conv_backward_entry("pccnn_conv_backward", false, basis, pts, feats, samples, neigh, ends, radii, weights,
                               in_grads, proj, mirror, grad_mask, n, m, t, d, c_in, num_mlps, c_out, divide_by_count,
                               d_weights, d_feats, d_param_a, d_param_b, d_pdf, d_pts, d_samples, workspace,
                               workspace_bytes, stream);
}

extern "C" int pccnn_conv_backward_bf16(const pccnn_basis *basis, const float *pts, const float *feats,
                                        const float *samples, const int32_t *neigh, const int32_t *ends,
                                        const float *radii, const float *weights, const float *in_grads,
                                        const uint16_t *proj, const int32_t *mirror, int grad_mask, int64_t n,
                                        int64_t m, int64_t t, int d, int c_in, int num_mlps, int c_out,
                                        int divide_by_count, float *d_weights, float *d_feats, float *d_param_a,
                                        float *d_param_b, float *d_pdf, float *d_pts, float *d_samples,
                                        void *workspace, size_t workspace_bytes, void *stream)
{
    return conv_backward_entry("pccnn_conv_backward_bf16", true, basis, pts, feats, samples, neigh, ends, radii,
                               weights, in_grads, proj, mirror, grad_mask, n, m, t, d, c_in, num_mlps, c_out,
                               divide_by_count, d_weights, d_feats, d_param_a, d_param_b, d_pdf, d_pts, d_samples,
                               workspace, workspace_bytes, stream);
}

extern "C" int pccnn_conv_weight_var(const pccnn_basis *basis, const float *pts, const float *feats,
                                     const float *samples, const int32_t *neigh, const int32_t *ends,
                                     const float *radii, int64_t n, int64_t m, int64_t t, int d, int c_in,
                                     int divide_by_count, float *out, void *workspace, size_t workspace_bytes,
                                     void *stream)
{
    ConvGeom g;
    int rc = basis_geom("pccnn_conv_weight_var", basis, pts, samples, neigh, ends, radii, n, m, t, c_in, g);
    if (rc != PCCNN_OK) return rc;
    if ((rc = conv_validate("pccnn_conv_weight_var", n, m, t, d, c_in, g.k, 1, 1)) != PCCNN_OK) return rc;
    const bool geom = basis->kind != PCCNN_BASIS_EXPLICIT;
    PCCNN_REQUIRE(feats && ends && out && (t == 0 || neigh) && (!geom || (pts && samples && radii)), PCCNN_ERR_INVALID,
                  "pccnn_conv_weight_var: null pointer");
    if (d != 3 && geom) {
        PCCNN_REQUIRE(pair_basis_kind(basis->kind), PCCNN_ERR_UNSUPPORTED,
                      "pccnn_conv_weight_var: basis kind %d needs 3 dimensions (d=%d)", basis->kind, d);
        size_t rest = 0;
        void *ws = ws_after(workspace, workspace_bytes, (size_t)(t > 0 ? t : 1) * g.k * sizeof(float), rest);
        PCCNN_REQUIRE(ws != nullptr, PCCNN_ERR_WORKSPACE, "pccnn_conv_weight_var: workspace of %zu bytes, need %zu",
                      workspace_bytes, pccnn_conv_weight_var_workspace_bytes(m, t, c_in, g.k));
        float *pair_w = (float *)workspace;
        const PairGeom pg = {pts, samples, (const int2 *)neigh, radii, basis->pdf, basis->a, basis->b, basis->sigma, t, d,
                             g.k};
        if ((rc = pair_basis_forward(basis->kind, pg, pair_w, (hipStream_t)stream)) != PCCNN_OK) return rc;
        ConvGeom ge = {nullptr, nullptr, (const int2 *)neigh, ends, nullptr, nullptr, pair_w, nullptr, 1.0f, n, m, t,
                       c_in, g.k};
        return conv_weight_var<BASIS_EXPLICIT>(ge, feats, out, ws, rest, (hipStream_t)stream, divide_by_count != 0);
    }
#define CALL(B) conv_weight_var<B>(g, feats, out, workspace, workspace_bytes, (hipStream_t)stream, divide_by_count != 0)
    BASIS_DISPATCH(basis->kind, CALL)
#undef CALL
}

extern "C" int pccnn_linear_basis_forward(const float *pts, const float *samples, const int32_t *neigh,
                                          const float *radii, const float *axis, const float *bias, int64_t n,
                                          int64_t m, int64_t t, int d, int k, float *basis_out, void *stream)
{
    int rc = conv_validate("pccnn_linear_basis_forward", n, m, t, d, 1, k, 1, 1);
    if (rc != PCCNN_OK || t == 0) return rc;
    PCCNN_REQUIRE(pts && samples && neigh && radii && axis && bias && basis_out, PCCNN_ERR_INVALID,
                  "pccnn_linear_basis_forward: null pointer");
    if (d != 3) {
        const PairGeom pg = {pts, samples, (const int2 *)neigh, radii, nullptr, axis, bias, 1.0f, t, d, k};
        return pair_basis_forward(PAIR_BASIS_LINEAR, pg, basis_out, (hipStream_t)stream);
    }
    ConvGeom g = {pts, samples, (const int2 *)neigh, nullptr, radii, nullptr, axis, bias, 1.0f, n, m, t, 1, k};
    linear_basis_fwd_kernel<<<(unsigned)pccnn_ceil_div(t * k, 256), 256, 0, (hipStream_t)stream>>>(g, basis_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" size_t pccnn_linear_basis_workspace_bytes(int64_t t)
{
    (void)t;
    return pccnn_align((size_t)(1024 + PARAM_REDUCE_GROUPS) * 256 * sizeof(float)) + 256;
}

extern "C" int pccnn_linear_basis_backward(const float *pts, const float *samples, const int32_t *neigh,
                                           const float *radii, const float *axis, const float *bias,
                                           const float *basis_grads, int64_t n, int64_t m, int64_t t, int d, int k,
                                           float *d_pts, float *d_samples, float *d_axis, float *d_bias,
                                           void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = conv_validate("pccnn_linear_basis_backward", n, m, t, d, 1, k, 1, 1);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(radii && axis && bias && d_axis && d_bias && (n == 0 || (pts && d_pts)) && (m == 0 || (samples && d_samples)) &&
                      (t == 0 || (neigh && basis_grads)),
                  PCCNN_ERR_INVALID, "pccnn_linear_basis_backward: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if ((rc = pccnn_fill_f32(d_pts, 0.0f, n * d, s)) != PCCNN_OK) return rc;
    if ((rc = pccnn_fill_f32(d_samples, 0.0f, m * d, s)) != PCCNN_OK) return rc;
    if (t == 0 || d != 3) {
        if ((rc = pccnn_fill_f32(d_axis, 0.0f, (int64_t)d * k, s)) != PCCNN_OK) return rc;
        if ((rc = pccnn_fill_f32(d_bias, 0.0f, k, s)) != PCCNN_OK || t == 0) return rc;
        const PairGeom pg = {pts, samples, (const int2 *)neigh, radii, nullptr, axis, bias, 1.0f, t, d, k};
        return pair_basis_backward(PAIR_BASIS_LINEAR, pg, basis_grads, d_pts, d_samples, nullptr, d_axis, d_bias, s);
    }
    const int kpad = kpad_of(k);
    int64_t blocks = pccnn_ceil_div(t, (int64_t)4 * (64 / kpad) * 8);
    if (blocks > 1024) blocks = 1024;
    PccnnArena arena(workspace, workspace_bytes);
    float *partials = arena.take<float>((size_t)(blocks + PARAM_REDUCE_GROUPS) * 256);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_linear_basis_backward: workspace of %zu bytes, need %zu",
                  workspace_bytes, pccnn_linear_basis_workspace_bytes(t));
    float *stage = partials + blocks * 256;
    ConvGeom g = {pts, samples, (const int2 *)neigh, nullptr, radii, nullptr, axis, bias, 1.0f, n, m, t, 1, k};
    switch (kpad) {
    case 8: linear_basis_bwd_kernel<8><<<(unsigned)blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, partials); break;
    case 16: linear_basis_bwd_kernel<16><<<(unsigned)blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, partials); break;
    case 32: linear_basis_bwd_kernel<32><<<(unsigned)blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, partials); break;
    default: linear_basis_bwd_kernel<64><<<(unsigned)blocks, 256, 0, s>>>(g, basis_grads, d_pts, d_samples, partials); break;
    }
    PCCNN_LAUNCH_CHECK();
    conv_param_reduce1_kernel<<<PARAM_REDUCE_GROUPS, 256, 0, s>>>(partials, blocks, stage);
    PCCNN_LAUNCH_CHECK();
    conv_param_reduce2_kernel<BASIS_MLP><<<1, 256, 0, s>>>(stage, PARAM_REDUCE_GROUPS, k, d_axis, d_bias);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" int pccnn_mirror_pairs(const int32_t *neigh, const int32_t *ends, int64_t t, int64_t m, int32_t *mirror_out,
                                  int32_t *missing_out, void *stream)
{
    PCCNN_REQUIRE(t >= 0 && m >= 0 && t < (1ll << 31) && m < (1ll << 31), PCCNN_ERR_INVALID,
                  "pccnn_mirror_pairs: t=%lld m=%lld", (long long)t, (long long)m);
    PCCNN_REQUIRE(missing_out && (t == 0 || (neigh && ends && mirror_out)), PCCNN_ERR_INVALID,
                  "pccnn_mirror_pairs: null pointer");
    hipStream_t s = (hipStream_t)stream;
    int rc = pccnn_fill_i32(missing_out, 0, 1, s);
    if (rc != PCCNN_OK || t == 0) return rc;
    mirror_pairs_kernel<<<(unsigned)pccnn_ceil_div(t, 256), 256, 0, s>>>((const int2 *)neigh, ends, t, m, mirror_out,
                                                                         missing_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}
