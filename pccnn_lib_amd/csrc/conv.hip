// KPConv / MCConv: basis projection and neighbor gather-aggregate (forward and backward), plus
// the host entry points that chain them with the fp32 MFMA contraction.
//
// Forward, per sample s:  P[s][f][k] = sum over the pairs t of s of  F[n_t][f] * w[t][k]
//   * one wavefront per (sample, block of 64 input features): lane l owns feature f = 64*fb + l
//     and keeps the K partial sums of its feature in registers;
//   * the pair geometry (neighbor id, normalised offset, density) of up to 64 pairs is loaded
//     lane-parallel, then pair by pair the basis values w[t][0..K) are evaluated by lanes 0..K-1
//     and handed to every lane as scalars (readlane), while the feature row of the neighbor is
//     one coalesced read;
//   * P is stored k-fastest, i.e. row f*K + k of the contraction, then out = P x W on MFMA.
// Backward: dP = dOut x W^T and dW = P^T x dOut on MFMA; a second per-sample walk turns dP into
// feature gradients (coalesced float atomics per neighbor row) and per-pair basis gradients
// (butterfly reduce-scatter across the lanes); a pair-parallel kernel then applies the basis
// derivative and accumulates point, sample, density and basis-parameter gradients.
#include "common.h"

enum { BASIS_KP = 0, BASIS_MLP = 1 };

struct ConvGeom {
    const float *pts;       // [n,3]
    const float *samples;   // [m,3]
    const int2 *neigh;      // [t] (point, sample)
    const int32_t *ends;    // [m]
    const float *radii;     // [3]
    const float *pdf;       // [n] (MLP) or null
    const float *basis_a;   // KP: kernel points [K,3]; MLP: axis [3,K]
    const float *basis_b;   // MLP: bias [K]
    float sigma;            // KP
    int64_t n, m, t;
    int c_in, k;
};

template <int BASIS> struct LaneBasis {
    float c0, c1, c2, c3;
    bool active;
    __device__ __forceinline__ void load(const ConvGeom &g, int k)
    {
        active = k < g.k;
        c0 = c1 = c2 = c3 = 0.0f;
        if (active) {
            if (BASIS == BASIS_KP) {
                c0 = g.basis_a[k * 3 + 0]; c1 = g.basis_a[k * 3 + 1]; c2 = g.basis_a[k * 3 + 2];
            } else {
                c0 = g.basis_a[k]; c1 = g.basis_a[g.k + k]; c2 = g.basis_a[2 * g.k + k]; c3 = g.basis_b[k];
            }
        }
    }
    // Basis value of this lane's k for a pair with normalised offset (dx,dy,dz).
    __device__ __forceinline__ float eval(float dx, float dy, float dz, float pdf, float sigma) const
    {
        float w;
        if (BASIS == BASIS_KP) {
            const float vx = c0 - dx, vy = c1 - dy, vz = c2 - dz;
            const float d2 = fmaxf(vx * vx + vy * vy + vz * vz, 0.0f);
            const float r = 1.0f - sqrtf(d2) / sigma;
            w = fminf(fmaxf(r, 0.0f), 1.0f);
        } else {
            float a = dx * c0 + dy * c1 + dz * c2 + c3;
            a = a > 0.0f ? a : a * 0.2f;
            w = a / pdf;
        }
        return active ? w : 0.0f;
    }
};

// ------------------------------------------------------------------------------- forward

template <int BASIS, int KPAD>
__global__ void __launch_bounds__(256)
conv_proj_fwd_kernel(ConvGeom g, const float *__restrict__ feats, float *__restrict__ proj)
{
    const int lane = pccnn_lane();
    const int64_t s = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (s >= g.m) return;                                           // wave-uniform
    const int f = blockIdx.y * 64 + lane;
    const bool fvalid = f < g.c_in;
    const int lo = s > 0 ? g.ends[s - 1] : 0;
    const int hi = g.ends[s];
    const float sx = g.samples[s * 3 + 0], sy = g.samples[s * 3 + 1], sz = g.samples[s * 3 + 2];
    const float ir0 = 1.0f / g.radii[0], ir1 = 1.0f / g.radii[1], ir2 = 1.0f / g.radii[2];
    LaneBasis<BASIS> lb;
    lb.load(g, lane % KPAD);

    float acc[KPAD];
#pragma unroll
    for (int k = 0; k < KPAD; ++k) acc[k] = 0.0f;

    for (int cb = lo; cb < hi; cb += 64) {
        const int t = cb + lane;
        int nidx = 0;
        float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
        if (t < hi) {
            nidx = g.neigh[t].x;
            dx = (g.pts[(int64_t)nidx * 3 + 0] - sx) * ir0;
            dy = (g.pts[(int64_t)nidx * 3 + 1] - sy) * ir1;
            dz = (g.pts[(int64_t)nidx * 3 + 2] - sz) * ir2;
            if (BASIS == BASIS_MLP) pd = g.pdf[nidx];
        }
        const int cnt = (hi - cb) < 64 ? (hi - cb) : 64;
        for (int j0 = 0; j0 < cnt; j0 += 4) {
            float row[4], wv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = j0 + u;
                row[u] = 0.0f;
                wv[u] = 0.0f;
                if (j < cnt) {                                      // uniform
                    const int bn = pccnn_bcast_i(nidx, j);
                    if (fvalid) row[u] = feats[(int64_t)bn * g.c_in + f];
                    wv[u] = lb.eval(pccnn_bcast_f(dx, j), pccnn_bcast_f(dy, j), pccnn_bcast_f(dz, j),
                                    pccnn_bcast_f(pd, j), g.sigma);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int k = 0; k < KPAD; ++k)
                    acc[k] += row[u] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv[u]), k));
            }
        }
    }
    if (fvalid) {
        float *dst = proj + ((int64_t)s * g.c_in + f) * g.k;
        if (g.k == KPAD && (KPAD % 4) == 0) {
#pragma unroll
            for (int k = 0; k < KPAD; k += 4) {
                float4 v = make_float4(acc[k], acc[k + 1], acc[k + 2], acc[k + 3]);
                *(float4 *)(dst + k) = v;
            }
        } else {
#pragma unroll
            for (int k = 0; k < KPAD; ++k)
                if (k < g.k) dst[k] = acc[k];
        }
    }
}

// ------------------------------------------------------------------------------ backward

// Sum p[k] over the 64 lanes for every k with log-step exchanges that halve the number of
// live values per lane at each step.  Returns, in every lane, the total for k = *k_out.
template <int KPAD>
__device__ __forceinline__ float reduce_scatter(float (&p)[KPAD], int lane, int &k_out)
{
    int kidx = 0;
    int mask = 32;
#pragma unroll
    for (int width = KPAD; width > 1; width >>= 1) {
        const int half = width >> 1;
        const bool upper = (lane & mask) != 0;
#pragma unroll
        for (int j = 0; j < half; ++j) {
            const float send = upper ? p[j] : p[j + half];
            const float keep = upper ? p[j + half] : p[j];
            p[j] = keep + __shfl_xor(send, mask);
        }
        if (upper) kidx += half;
        mask >>= 1;
    }
    float v = p[0];
    for (; mask > 0; mask >>= 1) v += __shfl_xor(v, mask);
    k_out = kidx;
    return v;
}

template <int KPAD> __host__ __device__ constexpr int reduce_scatter_owner_mask()
{
    // lanes whose low bits (those not consumed by the halving steps) are zero own the result
    return KPAD >= 64 ? 0 : (64 / KPAD) - 1;
}

template <int BASIS, int KPAD>
__global__ void __launch_bounds__(256)
conv_proj_bwd_kernel(ConvGeom g, const float *__restrict__ feats, const float *__restrict__ proj_grads,
                     float *__restrict__ feat_grads, float *__restrict__ basis_grads)
{
    const int lane = pccnn_lane();
    const int64_t s = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (s >= g.m) return;                                           // wave-uniform
    const int lo = s > 0 ? g.ends[s - 1] : 0;
    const int hi = g.ends[s];
    const float sx = g.samples[s * 3 + 0], sy = g.samples[s * 3 + 1], sz = g.samples[s * 3 + 2];
    const float ir0 = 1.0f / g.radii[0], ir1 = 1.0f / g.radii[1], ir2 = 1.0f / g.radii[2];
    LaneBasis<BASIS> lb;
    lb.load(g, lane % KPAD);
    const int fblocks = (g.c_in + 63) / 64;

    for (int fb = 0; fb < fblocks; ++fb) {
        const int f = fb * 64 + lane;
        const bool fvalid = f < g.c_in;
        float gp[KPAD];
#pragma unroll
        for (int k = 0; k < KPAD; ++k) gp[k] = 0.0f;
        if (fvalid) {
            const float *src = proj_grads + ((int64_t)s * g.c_in + f) * g.k;
            if (g.k == KPAD && (KPAD % 4) == 0) {
#pragma unroll
                for (int k = 0; k < KPAD; k += 4) {
                    const float4 v = *(const float4 *)(src + k);
                    gp[k] = v.x; gp[k + 1] = v.y; gp[k + 2] = v.z; gp[k + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int k = 0; k < KPAD; ++k)
                    if (k < g.k) gp[k] = src[k];
            }
        }
        for (int cb = lo; cb < hi; cb += 64) {
            const int t = cb + lane;
            int nidx = 0;
            float dx = 0.f, dy = 0.f, dz = 0.f, pd = 1.0f;
            if (t < hi) {
                nidx = g.neigh[t].x;
                dx = (g.pts[(int64_t)nidx * 3 + 0] - sx) * ir0;
                dy = (g.pts[(int64_t)nidx * 3 + 1] - sy) * ir1;
                dz = (g.pts[(int64_t)nidx * 3 + 2] - sz) * ir2;
                if (BASIS == BASIS_MLP) pd = g.pdf[nidx];
            }
            const int cnt = (hi - cb) < 64 ? (hi - cb) : 64;
            for (int j = 0; j < cnt; ++j) {
                const int bn = pccnn_bcast_i(nidx, j);
                const float row = fvalid ? feats[(int64_t)bn * g.c_in + f] : 0.0f;
                const float wv = lb.eval(pccnn_bcast_f(dx, j), pccnn_bcast_f(dy, j), pccnn_bcast_f(dz, j),
                                         pccnn_bcast_f(pd, j), g.sigma);
                float gf = 0.0f;
                float pk[KPAD];
#pragma unroll
                for (int k = 0; k < KPAD; ++k) {
                    gf += gp[k] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv), k));
                    pk[k] = gp[k] * row;
                }
                if (fvalid) unsafeAtomicAdd(&feat_grads[(int64_t)bn * g.c_in + f], gf);
                int kk;
                const float tot = reduce_scatter<KPAD>(pk, lane, kk);
                if ((lane & reduce_scatter_owner_mask<KPAD>()) == 0 && kk < g.k) {
                    float *dst = basis_grads + (int64_t)(cb + j) * g.k + kk;
                    *dst = (fb == 0) ? tot : (*dst + tot);
                }
            }
        }
    }
}

// One thread per pair: derivative of the basis w.r.t. its inputs and parameters.
// param_grads: KP -> d_kernel_pts [K,3];  MLP -> d_axis [3,K] followed by d_bias [K].
template <int BASIS>
__global__ void __launch_bounds__(256)
conv_basis_bwd_kernel(ConvGeom g, const float *__restrict__ basis_grads, float *__restrict__ d_pts,
                      float *__restrict__ d_samples, float *__restrict__ d_pdf, float *__restrict__ param_grads)
{
    // The KPConv correlation has a kink where a pair sits exactly one sigma away from a kernel
    // point, and every self pair (offset 0) does so for the kernel points closest to the centre.
    // Which side of the kink such a pair falls on is decided by the last bit of the fp32
    // distance, so the distance is evaluated exactly as written: no fused multiply-add.
#pragma clang fp contract(off)
    extern __shared__ float lds_param[];                            // 4*K floats
    const int nparam = (BASIS == BASIS_KP ? 3 : 4) * g.k;
    for (int i = threadIdx.x; i < nparam; i += blockDim.x) lds_param[i] = 0.0f;
    __syncthreads();
    const float ir0 = 1.0f / g.radii[0], ir1 = 1.0f / g.radii[1], ir2 = 1.0f / g.radii[2];
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < g.t; t += (int64_t)gridDim.x * blockDim.x) {
        const int2 pr = g.neigh[t];
        const float dx = (g.pts[(int64_t)pr.x * 3 + 0] - g.samples[(int64_t)pr.y * 3 + 0]) * ir0;
        const float dy = (g.pts[(int64_t)pr.x * 3 + 1] - g.samples[(int64_t)pr.y * 3 + 1]) * ir1;
        const float dz = (g.pts[(int64_t)pr.x * 3 + 2] - g.samples[(int64_t)pr.y * 3 + 2]) * ir2;
        float gx = 0.f, gy = 0.f, gz = 0.f, gpdf = 0.f;
        const float *gb = basis_grads + t * g.k;
        if (BASIS == BASIS_KP) {
            for (int k = 0; k < g.k; ++k) {
                const float vx = g.basis_a[k * 3 + 0] - dx, vy = g.basis_a[k * 3 + 1] - dy,
                            vz = g.basis_a[k * 3 + 2] - dz;
                const float dist = sqrtf(fmaxf(vx * vx + vy * vy + vz * vz, 0.0f));
                const float res = 1.0f - dist / g.sigma;
                if (res >= 0.0f) {
                    const float c = -(gb[k] / g.sigma) * (1.0f / (dist + 1e-6f));
                    const float cx = c * vx, cy = c * vy, cz = c * vz;
                    gx -= cx; gy -= cy; gz -= cz;
                    atomicAdd(&lds_param[k * 3 + 0], cx);
                    atomicAdd(&lds_param[k * 3 + 1], cy);
                    atomicAdd(&lds_param[k * 3 + 2], cz);
                }
            }
        } else {
            const float pd = g.pdf[pr.x];
            const float inv_pd = 1.0f / pd;
            for (int k = 0; k < g.k; ++k) {
                const float a0 = g.basis_a[k], a1 = g.basis_a[g.k + k], a2 = g.basis_a[2 * g.k + k];
                float act = dx * a0 + dy * a1 + dz * a2 + g.basis_b[k];
                const bool pos = act > 0.0f;
                act = pos ? act : act * 0.2f;
                const float gk = gb[k];
                gpdf -= act * gk * inv_pd * inv_pd;
                const float c = gk * inv_pd * (pos ? 1.0f : 0.2f);
                gx += c * a0; gy += c * a1; gz += c * a2;
                atomicAdd(&lds_param[k], dx * c);
                atomicAdd(&lds_param[g.k + k], dy * c);
                atomicAdd(&lds_param[2 * g.k + k], dz * c);
                atomicAdd(&lds_param[3 * g.k + k], c);
            }
            unsafeAtomicAdd(&d_pdf[pr.x], gpdf);
        }
        gx *= ir0; gy *= ir1; gz *= ir2;
        unsafeAtomicAdd(&d_pts[(int64_t)pr.x * 3 + 0], gx);
        unsafeAtomicAdd(&d_pts[(int64_t)pr.x * 3 + 1], gy);
        unsafeAtomicAdd(&d_pts[(int64_t)pr.x * 3 + 2], gz);
        unsafeAtomicAdd(&d_samples[(int64_t)pr.y * 3 + 0], -gx);
        unsafeAtomicAdd(&d_samples[(int64_t)pr.y * 3 + 1], -gy);
        unsafeAtomicAdd(&d_samples[(int64_t)pr.y * 3 + 2], -gz);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nparam; i += blockDim.x) unsafeAtomicAdd(&param_grads[i], lds_param[i]);
}

__global__ void copy_params_kernel(const float *__restrict__ src, float *__restrict__ dst_a, int count_a,
                                   float *__restrict__ dst_b, int count_b)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count_a) dst_a[i] = src[i];
    else if (i < count_a + count_b) dst_b[i - count_a] = src[i];
}

// ------------------------------------------------------------------------------- host side

static int kpad_of(int k) { return k <= 8 ? 8 : (k <= 16 ? 16 : (k <= 32 ? 32 : 64)); }

template <int BASIS>
static int launch_proj_fwd(const ConvGeom &g, const float *feats, float *proj, hipStream_t s)
{
    dim3 grid((unsigned)pccnn_ceil_div(g.m, 4), (unsigned)((g.c_in + 63) / 64));
    PccnnTimed timed(PCCNN_T_PROJ_FWD, s);
    switch (kpad_of(g.k)) {
    case 8: conv_proj_fwd_kernel<BASIS, 8><<<grid, 256, 0, s>>>(g, feats, proj); break;
    case 16: conv_proj_fwd_kernel<BASIS, 16><<<grid, 256, 0, s>>>(g, feats, proj); break;
    case 32: conv_proj_fwd_kernel<BASIS, 32><<<grid, 256, 0, s>>>(g, feats, proj); break;
    default: conv_proj_fwd_kernel<BASIS, 64><<<grid, 256, 0, s>>>(g, feats, proj); break;
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

template <int BASIS>
static int launch_proj_bwd(const ConvGeom &g, const float *feats, const float *proj_grads, float *feat_grads,
                           float *basis_grads, hipStream_t s)
{
    dim3 grid((unsigned)pccnn_ceil_div(g.m, 4));
    PccnnTimed timed(PCCNN_T_PROJ_BWD, s);
    switch (kpad_of(g.k)) {
    case 8: conv_proj_bwd_kernel<BASIS, 8><<<grid, 256, 0, s>>>(g, feats, proj_grads, feat_grads, basis_grads); break;
    case 16: conv_proj_bwd_kernel<BASIS, 16><<<grid, 256, 0, s>>>(g, feats, proj_grads, feat_grads, basis_grads); break;
    case 32: conv_proj_bwd_kernel<BASIS, 32><<<grid, 256, 0, s>>>(g, feats, proj_grads, feat_grads, basis_grads); break;
    default: conv_proj_bwd_kernel<BASIS, 64><<<grid, 256, 0, s>>>(g, feats, proj_grads, feat_grads, basis_grads); break;
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

static int conv_validate(const char *who, int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int num_mlps,
                         int c_out)
{
    PCCNN_REQUIRE(d == 3, PCCNN_ERR_UNSUPPORTED, "%s: d=%d is not supported (d must be 3)", who, d);
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
    if (!backward) return proj + 256;
    size_t basis_g = pccnn_align((size_t)t * k * sizeof(float));
    size_t splitk = pccnn_align((size_t)CONV_SPLIT_K * c_in * k * c_out * sizeof(float));
    return 2 * proj + basis_g + splitk + pccnn_align(4 * 64 * sizeof(float)) + 256;
}

// out[m, c_out] = P[m, c_in*k] x W, with the feature axis split over num_mlps independent
// weight blocks (num_mlps == 1 is the plain product).
static int contraction_fwd(const float *proj, const float *weights, float *out, int64_t m, int c_in, int k,
                           int num_mlps, int c_out, hipStream_t s)
{
    const int64_t inner = (int64_t)c_in * k / num_mlps;
    const int64_t co = c_out / num_mlps;
    return pccnn_gemm_f32(proj, weights, out, m, co, inner, 0, 0, (int64_t)c_in * k, co, c_out, num_mlps, inner,
                          inner * co, co, 1, nullptr, 0, s);
}

// d_proj[m, c_in*k] = dOut x W^T and d_weights = P^T x dOut.
static int contraction_bwd(const float *proj, const float *weights, const float *in_grads, float *d_proj,
                           float *d_weights, int64_t m, int c_in, int k, int num_mlps, int c_out, float *splitk_ws,
                           size_t splitk_bytes, hipStream_t s)
{
    const int64_t inner = (int64_t)c_in * k / num_mlps;
    const int64_t co = c_out / num_mlps;
    int rc = pccnn_gemm_f32(in_grads, weights, d_proj, m, inner, co, 0, 1, c_out, co, (int64_t)c_in * k, num_mlps,
                            co, inner * co, inner, 1, nullptr, 0, s);
    if (rc != PCCNN_OK) return rc;
    int split = (int)(m >= 4096 ? CONV_SPLIT_K : 1);
    return pccnn_gemm_f32(proj, in_grads, d_weights, inner, co, m, 1, 0, (int64_t)c_in * k, c_out, co, num_mlps,
                          inner, co, inner * co, split, splitk_ws, splitk_bytes, s);
}

template <int BASIS>
static int conv_forward(ConvGeom g, const float *feats, const float *weights, int num_mlps, int c_out, float *out,
                        void *workspace, size_t workspace_bytes, hipStream_t s)
{
    if (g.m == 0) return PCCNN_OK;
    PccnnArena arena(workspace, workspace_bytes);
    float *proj = arena.take<float>((size_t)g.m * g.c_in * g.k);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv forward: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 0));
    int rc = launch_proj_fwd<BASIS>(g, feats, proj, s);
    if (rc != PCCNN_OK) return rc;
    return contraction_fwd(proj, weights, out, g.m, g.c_in, g.k, num_mlps, c_out, s);
}

template <int BASIS>
static int conv_backward(ConvGeom g, const float *feats, const float *weights, const float *in_grads, int num_mlps,
                         int c_out, float *d_weights, float *d_feats, float *d_param_a, float *d_param_b,
                         float *d_pdf, float *d_pts, float *d_samples, void *workspace, size_t workspace_bytes,
                         hipStream_t s)
{
    // d_param_a: d_kernel_pts [K,3] (KP) or d_axis [3,K] (MLP); d_param_b: d_bias [K] (MLP only)
    const int count_a = 3 * g.k, count_b = (BASIS == BASIS_KP ? 0 : g.k);
    const int nparam = count_a + count_b;
    int rc;
    PccnnArena arena(workspace, workspace_bytes);
    float *d_param = arena.take<float>(4 * 64);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv backward: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 1));
    if ((rc = pccnn_fill_f32(d_feats, 0.0f, g.n * g.c_in, s)) != PCCNN_OK) return rc;
    if ((rc = pccnn_fill_f32(d_pts, 0.0f, g.n * 3, s)) != PCCNN_OK) return rc;
    if ((rc = pccnn_fill_f32(d_samples, 0.0f, g.m * 3, s)) != PCCNN_OK) return rc;
    if ((rc = pccnn_fill_f32(d_param, 0.0f, nparam, s)) != PCCNN_OK) return rc;
    if (d_pdf && (rc = pccnn_fill_f32(d_pdf, 0.0f, g.n, s)) != PCCNN_OK) return rc;
    if (g.m == 0 || g.t == 0) {
        if ((rc = pccnn_fill_f32(d_param_a, 0.0f, count_a, s)) != PCCNN_OK) return rc;
        if (count_b && (rc = pccnn_fill_f32(d_param_b, 0.0f, count_b, s)) != PCCNN_OK) return rc;
        return pccnn_fill_f32(d_weights, 0.0f, (int64_t)g.c_in * g.k * c_out / num_mlps, s);
    }

    float *proj = arena.take<float>((size_t)g.m * g.c_in * g.k);
    float *d_proj = arena.take<float>((size_t)g.m * g.c_in * g.k);
    float *basis_g = arena.take<float>((size_t)g.t * g.k);
    size_t splitk_elems = (size_t)CONV_SPLIT_K * g.c_in * g.k * c_out;
    float *splitk = arena.take<float>(splitk_elems);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "conv backward: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_conv_workspace_bytes(g.m, g.t, g.c_in, g.k, c_out, 1));
    if ((rc = launch_proj_fwd<BASIS>(g, feats, proj, s)) != PCCNN_OK) return rc;
    if ((rc = contraction_bwd(proj, weights, in_grads, d_proj, d_weights, g.m, g.c_in, g.k, num_mlps, c_out, splitk,
                              splitk_elems * sizeof(float), s)) != PCCNN_OK)
        return rc;
    if ((rc = launch_proj_bwd<BASIS>(g, feats, d_proj, d_feats, basis_g, s)) != PCCNN_OK) return rc;
    int64_t blocks = pccnn_ceil_div(g.t, 256);
    if (blocks > 2048) blocks = 2048;
    {
        PccnnTimed timed(PCCNN_T_BASIS_BWD, s);
        conv_basis_bwd_kernel<BASIS><<<(unsigned)blocks, 256, 4 * g.k * sizeof(float), s>>>(g, basis_g, d_pts, d_samples,
                                                                                            d_pdf, d_param);
    }
    PCCNN_LAUNCH_CHECK();
    copy_params_kernel<<<1, 256, 0, s>>>(d_param, d_param_a, count_a, d_param_b, count_b);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" int pccnn_kpconv_forward(const float *pts, const float *feats, const float *samples, const int32_t *neigh,
                                    const int32_t *ends, const float *radii, const float *kernel_pts, float sigma,
                                    const float *weights, int64_t n, int64_t m, int64_t t, int d, int c_in, int k,
                                    int c_out, float *out, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = conv_validate("pccnn_kpconv_forward", n, m, t, d, c_in, k, 1, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(sigma > 0.0f, PCCNN_ERR_INVALID, "pccnn_kpconv_forward: sigma=%g", sigma);
    PCCNN_REQUIRE(m == 0 || (pts && feats && samples && ends && radii && kernel_pts && weights && out && (t == 0 || neigh)),
                  PCCNN_ERR_INVALID, "pccnn_kpconv_forward: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, nullptr, kernel_pts, nullptr, sigma, n, m, t, c_in, k};
    return conv_forward<BASIS_KP>(g, feats, weights, 1, c_out, out, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int pccnn_kpconv_backward(const float *pts, const float *feats, const float *samples,
                                     const int32_t *neigh, const int32_t *ends, const float *radii,
                                     const float *kernel_pts, float sigma, const float *weights,
                                     const float *in_grads, int64_t n, int64_t m, int64_t t, int d, int c_in, int k,
                                     int c_out, float *d_weights, float *d_feats, float *d_kernel_pts, float *d_pts,
                                     float *d_samples, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = conv_validate("pccnn_kpconv_backward", n, m, t, d, c_in, k, 1, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(sigma > 0.0f, PCCNN_ERR_INVALID, "pccnn_kpconv_backward: sigma=%g", sigma);
    PCCNN_REQUIRE(d_weights && d_kernel_pts && kernel_pts && weights && radii && (n == 0 || (d_feats && d_pts && pts && feats)) &&
                      (m == 0 || (d_samples && samples && ends && in_grads)) && (t == 0 || neigh),
                  PCCNN_ERR_INVALID, "pccnn_kpconv_backward: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, nullptr, kernel_pts, nullptr, sigma, n, m, t, c_in, k};
    return conv_backward<BASIS_KP>(g, feats, weights, in_grads, 1, c_out, d_weights, d_feats, d_kernel_pts, nullptr,
                                   nullptr, d_pts, d_samples, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int pccnn_mcconv_forward(const float *pts, const float *pdf, const float *feats, const float *samples,
                                    const int32_t *neigh, const int32_t *ends, const float *radii, const float *axis,
                                    const float *bias, const float *weights, int64_t n, int64_t m, int64_t t, int d,
                                    int c_in, int k, int num_mlps, int c_out, float *out, void *workspace,
                                    size_t workspace_bytes, void *stream)
{
    int rc = conv_validate("pccnn_mcconv_forward", n, m, t, d, c_in, k, num_mlps, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(m == 0 || (pts && pdf && feats && samples && ends && radii && axis && bias && weights && out &&
                             (t == 0 || neigh)),
                  PCCNN_ERR_INVALID, "pccnn_mcconv_forward: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, pdf, axis, bias, 1.0f, n, m, t, c_in, k};
    return conv_forward<BASIS_MLP>(g, feats, weights, num_mlps, c_out, out, workspace, workspace_bytes,
                                   (hipStream_t)stream);
}

extern "C" int pccnn_mcconv_backward(const float *pts, const float *pdf, const float *feats, const float *samples,
                                     const int32_t *neigh, const int32_t *ends, const float *radii,
                                     const float *axis, const float *bias, const float *weights,
                                     const float *in_grads, int64_t n, int64_t m, int64_t t, int d, int c_in, int k,
                                     int num_mlps, int c_out, float *d_weights, float *d_feats, float *d_axis,
                                     float *d_bias, float *d_pdf, float *d_pts, float *d_samples, void *workspace,
                                     size_t workspace_bytes, void *stream)
{
    int rc = conv_validate("pccnn_mcconv_backward", n, m, t, d, c_in, k, num_mlps, c_out);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(d_weights && d_axis && d_bias && axis && bias && weights && radii &&
                      (n == 0 || (d_feats && d_pts && d_pdf && pts && pdf && feats)) &&
                      (m == 0 || (d_samples && samples && ends && in_grads)) && (t == 0 || neigh),
                  PCCNN_ERR_INVALID, "pccnn_mcconv_backward: null pointer");
    ConvGeom g = {pts, samples, (const int2 *)neigh, ends, radii, pdf, axis, bias, 1.0f, n, m, t, c_in, k};
    return conv_backward<BASIS_MLP>(g, feats, weights, in_grads, num_mlps, c_out, d_weights, d_feats, d_axis, d_bias,
                                    d_pdf, d_pts, d_samples, workspace, workspace_bytes, (hipStream_t)stream);
}
