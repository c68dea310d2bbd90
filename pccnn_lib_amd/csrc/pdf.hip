// Gaussian kernel density estimate over a neighbor list, and its gradient w.r.t. the points.
// A group of G lanes owns one sample: the lanes stride over the sample's pair segment
// (coalesced reads of the pair list, gathered reads of the neighbor coordinates), then a
// shuffle reduction inside the group produces the sample's density.
#include <math.h>

#include "common.h"

// fp32 expressions in this file must round exactly as written (no fused multiply-add).
#pragma clang fp contract(off)

template <int G, bool GRADS, int D>
__global__ void __launch_bounds__(256)
pdf_kernel(double norm_const, const float *__restrict__ bandwidth, const float *__restrict__ pts,
           const float *__restrict__ samples, int64_t n, const int2 *__restrict__ neigh,
           const int32_t *__restrict__ ends, const float *__restrict__ in_grads, float *__restrict__ out)
{
    // `samples` holds the coordinates of sample gid, `pts` the array the pair list's point column indexes;
    // they are the same array unless the caller searched in sorted-index space.
    const int64_t gid = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / G;
    const int sub = threadIdx.x % G;
    const bool valid = gid < n;
    float ib[D];
    float prod = 1.0f;
#pragma unroll
    for (int i = 0; i < D; ++i) {
        ib[i] = __fdiv_rn(1.0f, bandwidth[i]);
        prod = prod * ib[i];
    }
    // (prod of inverse bandwidths, fp32) * 1/pow(2*3.1415, m/2) in double
    const double scale = (double)prod * norm_const;
    int lo = 0, hi = 0;
    float c[D], g = 0.f;
#pragma unroll
    for (int i = 0; i < D; ++i) c[i] = 0.f;
    if (valid) {
        lo = gid > 0 ? ends[gid - 1] : 0;
        hi = ends[gid];
#pragma unroll
        for (int i = 0; i < D; ++i) c[i] = samples[gid * D + i];
        if (GRADS) g = in_grads[gid];
    }
    double acc = 0.0;
    float gsum[D];
#pragma unroll
    for (int i = 0; i < D; ++i) gsum[i] = 0.f;
    for (int t = lo + sub; t < hi; t += G) {
        const int j = neigh[t].x;
        float diff[D];
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < D; ++i) {
            diff[i] = (pts[(int64_t)j * D + i] - c[i]) * ib[i];
            dot = dot + diff[i] * diff[i];
        }
        const float e = expf(dot * (-0.5f));
        const double term = scale * (double)e;
        if (!GRADS) {
            acc += term;
        } else {
            const float local = (float)term;
#pragma unroll
            for (int i = 0; i < D; ++i) {
                const float lg = diff[i] * ib[i] * g * local;
                gsum[i] += lg;
                unsafeAtomicAdd(&out[(int64_t)j * D + i], -lg);
            }
        }
    }
    if (!GRADS) {
#pragma unroll
        for (int o = G / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
        if (valid && sub == 0) out[gid] = (float)acc;
    } else {
#pragma unroll
        for (int i = 0; i < D; ++i) {
#pragma unroll
            for (int o = G / 2; o > 0; o >>= 1) gsum[i] += __shfl_xor(gsum[i], o);
            if (valid && sub == 0) unsafeAtomicAdd(&out[gid * D + i], gsum[i]);
        }
    }
}

template <bool GRADS, int D>
static int pdf_launch_d(int manifold_dims, const float *bandwidth, const float *pts, const float *samples, int64_t n,
                        const int32_t *neigh, int64_t t, const int32_t *ends, const float *in_grads, float *out,
                        hipStream_t s)
{
    const double norm_const = 1.0 / pow(2.0 * 3.1415, (double)(float)manifold_dims / 2.0);
    const int64_t avg = n > 0 ? t / n : 0;
    const int2 *nb = (const int2 *)neigh;
    PccnnTimed timed(PCCNN_T_PDF, s);
#define PDF_GO(G)                                                                                            \
    pdf_kernel<G, GRADS, D><<<(unsigned)pccnn_ceil_div(n * G, 256), 256, 0, s>>>(norm_const, bandwidth, pts, samples, n, \
                                                                                 nb, ends, in_grads, out)
    if (avg <= 6) PDF_GO(4);
    else if (avg <= 12) PDF_GO(8);
    else if (avg <= 24) PDF_GO(16);
    else if (avg <= 48) PDF_GO(32);
    else PDF_GO(64);
#undef PDF_GO
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

template <bool GRADS>
static int pdf_launch(int d, int manifold_dims, const float *bandwidth, const float *pts, const float *samples,
                      int64_t n, const int32_t *neigh, int64_t t, const int32_t *ends, const float *in_grads,
                      float *out, hipStream_t s)
{
    switch (d) {
    case 2: return pdf_launch_d<GRADS, 2>(manifold_dims, bandwidth, pts, samples, n, neigh, t, ends, in_grads, out, s);
    case 3: return pdf_launch_d<GRADS, 3>(manifold_dims, bandwidth, pts, samples, n, neigh, t, ends, in_grads, out, s);
    case 4: return pdf_launch_d<GRADS, 4>(manifold_dims, bandwidth, pts, samples, n, neigh, t, ends, in_grads, out, s);
    case 5: return pdf_launch_d<GRADS, 5>(manifold_dims, bandwidth, pts, samples, n, neigh, t, ends, in_grads, out, s);
    default: return pdf_launch_d<GRADS, 6>(manifold_dims, bandwidth, pts, samples, n, neigh, t, ends, in_grads, out, s);
    }
}

static int pdf_validate(const char *who, const float *bandwidth, const float *pts, int64_t n, int d,
                        const int32_t *neigh, int64_t t, const int32_t *ends, const float *out)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED, "%s: d=%d is not supported (2 <= d <= 6)", who, d);
    PCCNN_REQUIRE(n >= 0 && t >= 0 && n < (1ll << 31) && t < (1ll << 31), PCCNN_ERR_INVALID, "%s: n=%lld t=%lld", who,
                  (long long)n, (long long)t);
    PCCNN_REQUIRE(n == 0 || (bandwidth && pts && ends && out), PCCNN_ERR_INVALID, "%s: null pointer", who);
    PCCNN_REQUIRE(t == 0 || neigh, PCCNN_ERR_INVALID, "%s: null neighbor list", who);
    return PCCNN_OK;
}

extern "C" int pccnn_compute_pdf(int manifold_dims, const float *bandwidth, const float *pts, int64_t n, int d,
                                 const int32_t *neigh, int64_t t, const int32_t *ends, float *pdf_out, void *stream)
{
    int rc = pdf_validate("pccnn_compute_pdf", bandwidth, pts, n, d, neigh, t, ends, pdf_out);
    if (rc != PCCNN_OK || n == 0) return rc;
    return pdf_launch<false>(d, manifold_dims, bandwidth, pts, pts, n, neigh, t, ends, nullptr, pdf_out,
                             (hipStream_t)stream);
}

extern "C" int pccnn_compute_pdf_sorted(int manifold_dims, const float *bandwidth, const float *pts_sorted,
                                        const float *samples, int64_t n, int d, const int32_t *neigh_sorted, int64_t t,
                                        const int32_t *ends, float *pdf_out, void *stream)
{
    int rc = pdf_validate("pccnn_compute_pdf_sorted", bandwidth, pts_sorted, n, d, neigh_sorted, t, ends, pdf_out);
    if (rc != PCCNN_OK || n == 0) return rc;
    PCCNN_REQUIRE(samples, PCCNN_ERR_INVALID, "pccnn_compute_pdf_sorted: null samples");
    return pdf_launch<false>(d, manifold_dims, bandwidth, pts_sorted, samples, n, neigh_sorted, t, ends, nullptr, pdf_out,
                             (hipStream_t)stream);
}

extern "C" int pccnn_compute_pdf_grads(int manifold_dims, const float *bandwidth, const float *pts, int64_t n,
                                       int d, const int32_t *neigh, int64_t t, const int32_t *ends,
                                       const float *in_grads, float *pt_grads_out, void *stream)
{
    int rc = pdf_validate("pccnn_compute_pdf_grads", bandwidth, pts, n, d, neigh, t, ends, pt_grads_out);
    if (rc != PCCNN_OK || n == 0) return rc;
    PCCNN_REQUIRE(in_grads, PCCNN_ERR_INVALID, "pccnn_compute_pdf_grads: null in_grads");
    rc = pccnn_fill_f32(pt_grads_out, 0.0f, n * d, (hipStream_t)stream);
    if (rc != PCCNN_OK) return rc;
    return pdf_launch<true>(d, manifold_dims, bandwidth, pts, pts, n, neigh, t, ends, in_grads, pt_grads_out,
                            (hipStream_t)stream);
}
