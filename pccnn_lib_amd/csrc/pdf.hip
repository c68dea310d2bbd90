// Gaussian kernel density estimate over a neighbor list, and its gradient w.r.t. the points.
// A group of G lanes owns one sample: the lanes stride over the sample's pair segment
// (coalesced reads of the pair list, gathered reads of the neighbor coordinates), then a
// shuffle reduction inside the group produces the sample's density.
#include <math.h>

#include "common.h"

// fp32 expressions in this file must round exactly as written (no fused multiply-add).
#pragma clang fp contract(off)

template <int G, bool GRADS>
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
    const float ib0 = __fdiv_rn(1.0f, bandwidth[0]);
    const float ib1 = __fdiv_rn(1.0f, bandwidth[1]);
    const float ib2 = __fdiv_rn(1.0f, bandwidth[2]);
    // (prod of inverse bandwidths, fp32) * 1/pow(2*3.1415, m/2) in double
    const double scale = (double)(1.0f * ib0 * ib1 * ib2) * norm_const;
    int lo = 0, hi = 0;
    float cx = 0.f, cy = 0.f, cz = 0.f, g = 0.f;
    if (valid) {
        lo = gid > 0 ? ends[gid - 1] : 0;
        hi = ends[gid];
        cx = samples[gid * 3 + 0];
        cy = samples[gid * 3 + 1];
        cz = samples[gid * 3 + 2];
        if (GRADS) g = in_grads[gid];
    }
    double acc = 0.0;
    float gx = 0.f, gy = 0.f, gz = 0.f;
    for (int t = lo + sub; t < hi; t += G) {
        const int j = neigh[t].x;
        const float dx = (pts[(int64_t)j * 3 + 0] - cx) * ib0;
        const float dy = (pts[(int64_t)j * 3 + 1] - cy) * ib1;
        const float dz = (pts[(int64_t)j * 3 + 2] - cz) * ib2;
        const float dot = dx * dx + dy * dy + dz * dz;
        const float e = expf(dot * (-0.5f));
        const double term = scale * (double)e;
        if (!GRADS) {
            acc += term;
        } else {
            const float local = (float)term;
            const float lx = dx * ib0 * g * local, ly = dy * ib1 * g * local, lz = dz * ib2 * g * local;
            gx += lx; gy += ly; gz += lz;
            unsafeAtomicAdd(&out[(int64_t)j * 3 + 0], -lx);
            unsafeAtomicAdd(&out[(int64_t)j * 3 + 1], -ly);
            unsafeAtomicAdd(&out[(int64_t)j * 3 + 2], -lz);
        }
    }
    if (!GRADS) {
#pragma unroll
        for (int o = G / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
        if (valid && sub == 0) out[gid] = (float)acc;
    } else {
#pragma unroll
        for (int o = G / 2; o > 0; o >>= 1) {
            gx += __shfl_xor(gx, o);
            gy += __shfl_xor(gy, o);
            gz += __shfl_xor(gz, o);
        }
        if (valid && sub == 0) {
            unsafeAtomicAdd(&out[gid * 3 + 0], gx);
            unsafeAtomicAdd(&out[gid * 3 + 1], gy);
            unsafeAtomicAdd(&out[gid * 3 + 2], gz);
        }
    }
}

template <bool GRADS>
static int pdf_launch(int manifold_dims, const float *bandwidth, const float *pts, const float *samples, int64_t n,
                      const int32_t *neigh, int64_t t, const int32_t *ends, const float *in_grads, float *out,
                      hipStream_t s)
{
    const double norm_const = 1.0 / pow(2.0 * 3.1415, (double)(float)manifold_dims / 2.0);
    const int64_t avg = n > 0 ? t / n : 0;
    const int2 *nb = (const int2 *)neigh;
    PccnnTimed timed(PCCNN_T_PDF, s);
#define PDF_GO(G)                                                                                         \
    pdf_kernel<G, GRADS><<<(unsigned)pccnn_ceil_div(n * G, 256), 256, 0, s>>>(norm_const, bandwidth, pts, samples, n, \
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

static int pdf_validate(const char *who, const float *bandwidth, const float *pts, int64_t n, int d,
                        const int32_t *neigh, int64_t t, const int32_t *ends, const float *out)
{
    PCCNN_REQUIRE(d == 3, PCCNN_ERR_UNSUPPORTED, "%s: d=%d is not supported (d must be 3)", who, d);
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
    return pdf_launch<false>(manifold_dims, bandwidth, pts, pts, n, neigh, t, ends, nullptr, pdf_out,
                             (hipStream_t)stream);
}

extern "C" int pccnn_compute_pdf_sorted(int manifold_dims, const float *bandwidth, const float *pts_sorted,
                                        const float *samples, int64_t n, int d, const int32_t *neigh_sorted, int64_t t,
                                        const int32_t *ends, float *pdf_out, void *stream)
{
    int rc = pdf_validate("pccnn_compute_pdf_sorted", bandwidth, pts_sorted, n, d, neigh_sorted, t, ends, pdf_out);
    if (rc != PCCNN_OK || n == 0) return rc;
    PCCNN_REQUIRE(samples, PCCNN_ERR_INVALID, "pccnn_compute_pdf_sorted: null samples");
    return pdf_launch<false>(manifold_dims, bandwidth, pts_sorted, samples, n, neigh_sorted, t, ends, nullptr, pdf_out,
                             (hipStream_t)stream);
}

extern "C" int pccnn_compute_pdf_grads(int manifold_dims, const float *bandwidth, const float *pts, int64_t n,
                                       int d, const int32_t *neigh, int64_t t, const int32_t *ends,
                                       const float *in_grads, float *pt_grads_out, void *stream)
{
    int rc = pdf_validate("pccnn_compute_pdf_grads", bandwidth, pts, n, d, neigh, t, ends, pt_grads_out);
    if (rc != PCCNN_OK || n == 0) return rc;
    PCCNN_REQUIRE(in_grads, PCCNN_ERR_INVALID, "pccnn_compute_pdf_grads: null in_grads");
    rc = pccnn_fill_f32(pt_grads_out, 0.0f, n * 3, (hipStream_t)stream);
    if (rc != PCCNN_OK) return rc;
    return pdf_launch<true>(manifold_dims, bandwidth, pts, pts, n, neigh, t, ends, in_grads, pt_grads_out,
                            (hipStream_t)stream);
}
