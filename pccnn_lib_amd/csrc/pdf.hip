// Gaussian kernel density estimate over a neighbor list, and its gradient w.r.t. the points.
// A group of G lanes owns one sample: the lanes stride over the sample's pair segment
// (coalesced reads of the pair list, gathered reads of the neighbor coordinates), then a
// shuffle reduction inside the group produces the sample's density.
#include <math.h>

#include "common.h"
#include "grid_walk.h"

// fp32 expressions in this file must round exactly as written (no fused multiply-add).
#pragma clang fp contract(off)

#ifndef PDF_XCD_CHUNK
#define PDF_XCD_CHUNK 64                   // consecutive workgroups of the grid walk that share an XCD
#endif

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

// ------------------------------------------------------------------- density straight from the grid
// Pointcloud.compute_pdf of the reference (pccnn_lib/pc/Pointcloud.py:81-109) builds a neighbor list with radius
// 4 x bandwidth and at most 300 neighbors only to sum a Gaussian over it and drop it.  Here one lane per point walks
// the 3 x 3 pillar ranges around its cell (the walk of the neighbor search, same order, same fp32 predicate) and adds
// the kernel values as it goes: no pair list, no count / scan / fill, no host read-back of the pair count.  A point
// with more hits than the cap walks a second time and keeps the subset the capped neighbor search keeps (hit number
// r iff floor((r + 1) cap / raw) > floor(r cap / raw)), so both routes sum the same terms.  The order of the
// additions is the same only in the one-lane kernels; the kernels that share a point between several lanes add
// strided partial sums, and the routes agree because the sums are kept in double, not bit for bit.
struct PdfGridArgs {
    const float *pts;          // [n,3] in key order
    const int64_t *keys;       // [n] sorted
    const int32_t *order;      // nullable [n]: original index of sorted point i
    GridRef grid;
    const int32_t *num_cells;  // [3]
    const float *radii;        // [3] search radii (= cell size)
    const float *bandwidth;    // [3]
    double norm_const;
    int max_neighbors;
    float *out;                // [n] in original order
    float *out_norm;           // nullable [n]: out divided by the number of points of the point's cloud
    int64_t n;
};

// Number of points of cloud b: its keys are the range [b * cells, (b + 1) * cells) of the sorted keys.
__device__ __forceinline__ int pdf_grid_cloud_count(const PdfGridArgs &a, long long b, long long cells)
{
    const long long k_lo = b * cells, k_hi = k_lo + cells;
    if (a.grid.cell_table && k_hi <= a.grid.total_cells) return a.grid.cell_table[k_hi] - a.grid.cell_table[k_lo];
    int64_t bound[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const long long want = e == 0 ? k_lo : k_hi;        // first index whose key is >= want
        int64_t lb = 0, ub = a.n;
        while (lb < ub) {
            const int64_t mid = (lb + ub) >> 1;
            if (a.keys[mid] < want) lb = mid + 1; else ub = mid;
        }
        bound[e] = lb;
    }
    return (int)(bound[1] - bound[0]);
}

#define PDF_GRID_UNROLL 4

// QUARTER: the search radius is exactly four bandwidths on every axis (what Pointcloud.compute_pdf asks for), i.e.
// 1 / radius == (1 / bandwidth) / 4 bit for bit.  Scaling by a power of two is exact, so the kernel's argument
// ((p - s) / bandwidth)^2 is then 16 x the predicate's ((s - p) / radius)^2, rounding included, and is not computed
// a second time.
template <bool CAPPED, bool QUARTER>
__device__ __forceinline__ void pdf_grid_walk(const PdfGridArgs &a, const int2 (*ranges)[64], int lane, int nr, bool go,
                                              float sx, float sy, float sz, const float (&ir)[3], const float (&ib)[3],
                                              double scale, int raw, int step, double &sum, int &cnt)
{
    int r = 0, j = 0, first = 0, len = 0, err = 0;
    bool active = go && nr > 0;
    if (active) {
        const int2 g = ranges[0][lane];
        first = g.x;
        len = g.y;
    }
    while (__any(active)) {
        if (active) {
            const int idx = first + j;
            const int left = len - j;
            float px[PDF_GRID_UNROLL], py[PDF_GRID_UNROLL], pz[PDF_GRID_UNROLL];
#pragma unroll
            for (int u = 0; u < PDF_GRID_UNROLL; ++u) {
                const int64_t iu = idx + (u < left ? u : 0);
                px[u] = a.pts[iu * 3 + 0];
                py[u] = a.pts[iu * 3 + 1];
                pz[u] = a.pts[iu * 3 + 2];
            }
#pragma unroll
            for (int u = 0; u < PDF_GRID_UNROLL; ++u) {
                // the predicate of the neighbor search: ((s - p) / r)^2 summed x, y, z in fp32, below 1
                const float vx = (sx - px[u]) * ir[0];
                const float vy = (sy - py[u]) * ir[1];
                const float vz = (sz - pz[u]) * ir[2];
                const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                if (u < left && acc < 1.0f) {
                    bool take = true;
                    if (CAPPED) {
                        err += step;
                        take = err >= raw;
                        if (take) err -= raw;
                    }
                    if (take) {
                        // the term of pdf_kernel: ((p - s) / bandwidth)^2 summed in fp32, exp in fp32, scaled in double
                        float dot;
                        if (QUARTER) {
                            dot = acc * 16.0f;
                        } else {
                            const float d0 = (px[u] - sx) * ib[0];
                            const float d1 = (py[u] - sy) * ib[1];
                            const float d2 = (pz[u] - sz) * ib[2];
                            dot = ((0.0f + d0 * d0) + d1 * d1) + d2 * d2;
                        }
                        sum += scale * (double)expf(dot * (-0.5f));
                    }
                    ++cnt;
                }
            }
            j += PDF_GRID_UNROLL;
            if (j >= len) {
                j = 0;
                if (++r < nr) {
                    const int2 g = ranges[r][lane];
                    first = g.x;
                    len = g.y;
                } else {
                    active = false;
                }
            }
        }
    }
}

__global__ void __launch_bounds__(256)
pdf_grid_kernel(PdfGridArgs a)
{
    __shared__ int2 ranges[4][9][64];          // written and read by the same lane only
    const int lane = pccnn_lane();
    const int wib = threadIdx.x >> 6;
    // (the points are in key order: an XCD gets one contiguous run of them)
    const int64_t base = ((pccnn_xcd_block(blockIdx.x, gridDim.x, PDF_XCD_CHUNK) * 256 + threadIdx.x) >> 6) * 64;
    if (base >= a.n) return;                   // wave-uniform
    const int64_t i = base + lane;
    const bool valid = i < a.n;
    long long key = -1;
    float sx = 0.f, sy = 0.f, sz = 0.f;
    if (valid) {
        key = a.keys[i];
        sx = a.pts[i * 3 + 0];
        sy = a.pts[i * 3 + 1];
        sz = a.pts[i * 3 + 2];
    }
    const int nc0 = a.num_cells[0], nc1 = a.num_cells[1], nc2 = a.num_cells[2];
    float ir[3], ib[3];
    float prod = 1.0f;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
        ir[c] = __fdiv_rn(1.0f, a.radii[c]);
        ib[c] = __fdiv_rn(1.0f, a.bandwidth[c]);
        prod = prod * ib[c];
    }
    const double scale = (double)prod * a.norm_const;
    const bool usable = valid && key >= 0;
    long long k = usable ? key : 0;
    const int c2 = (int)(k % nc2); k /= nc2;
    const int c1 = (int)(k % nc1);
    const long long pil = k; k /= nc1;
    const int c0 = (int)(k % nc0);
    int nr = 0;
    if (usable) {
        const int cmin = c2 > 0 ? c2 - 1 : 0, cmax = c2 + 1 < nc2 ? c2 + 1 : nc2 - 1;
#pragma unroll
        for (int o = 0; o < 9; ++o) {
            const int dx = o / 3 - 1, dy = o % 3 - 1;
            const int x = c0 + dx, y = c1 + dy;
            if (x >= 0 && x < nc0 && y >= 0 && y < nc1) {
                int first, len;
                grid_pillar_range(a.grid, pil + (long long)dx * nc1 + dy, nc2, cmin, cmax, first, len);
                if (len > 0) {
                    ranges[wib][nr][lane] = make_int2(first, len);
                    ++nr;
                }
            }
        }
    }
    double sum = 0.0;
    int cnt = 0;
    const bool quarter = ir[0] * 4.0f == ib[0] && ir[1] * 4.0f == ib[1] && ir[2] * 4.0f == ib[2];     // uniform
    if (quarter) pdf_grid_walk<false, true>(a, ranges[wib], lane, nr, usable, sx, sy, sz, ir, ib, scale, 0, 0, sum, cnt);
    else pdf_grid_walk<false, false>(a, ranges[wib], lane, nr, usable, sx, sy, sz, ir, ib, scale, 0, 0, sum, cnt);
    const bool redo = a.max_neighbors > 0 && cnt > a.max_neighbors;
    if (__any(redo)) {
        double capped_sum = 0.0;
        int again = 0;
        pdf_grid_walk<true, false>(a, ranges[wib], lane, nr, redo, sx, sy, sz, ir, ib, scale, cnt, a.max_neighbors,
                                   capped_sum, again);
        if (redo) sum = capped_sum;
    }
    if (valid) {
        const int64_t at = a.order ? (int64_t)a.order[i] : i;
        const float v = (float)sum;
        a.out[at] = v;
        if (a.out_norm) {
            // Pointcloud.py:105-109: the estimate divided by the cloud's point count, both as fp32
            const long long cells = (long long)nc0 * nc1 * nc2;
            const int count = usable ? pdf_grid_cloud_count(a, key / cells, cells) : 1;
            a.out_norm[at] = __fdiv_rn(v, (float)count);
        }
    }
}

// The same with G lanes per point, for clouds too small to fill the chip with one point per lane: the lanes of a
// group stride over every pillar range together, one candidate per lane and step, a ballot over the group counts
// and ranks the hits of the step (so the capped subset is the one of the one-lane walk), every lane sums its own
// hits in double and the group's sums are added at the end.
template <int G>
__global__ void __launch_bounds__(256)
pdf_grid_group_kernel(PdfGridArgs a)
{
    constexpr int GROUPS = 64 / G;
    __shared__ int2 ranges[4][GROUPS][9];
    const int lane = pccnn_lane();
    const int wib = threadIdx.x >> 6;
    const int grp = lane / G, sub = lane % G;
    const int64_t wave = (pccnn_xcd_block(blockIdx.x, gridDim.x, PDF_XCD_CHUNK) * 256 + threadIdx.x) >> 6;
    if (wave * GROUPS >= a.n) return;                 // wave-uniform
    const int64_t i = wave * GROUPS + grp;
    const bool valid = i < a.n;
    long long key = -1;
    float sx = 0.f, sy = 0.f, sz = 0.f;
    if (valid) {
        key = a.keys[i];
        sx = a.pts[i * 3 + 0];
        sy = a.pts[i * 3 + 1];
        sz = a.pts[i * 3 + 2];
    }
    const int nc0 = a.num_cells[0], nc1 = a.num_cells[1], nc2 = a.num_cells[2];
    float ir[3], ib[3];
    float prod = 1.0f;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
        ir[c] = __fdiv_rn(1.0f, a.radii[c]);
        ib[c] = __fdiv_rn(1.0f, a.bandwidth[c]);
        prod = prod * ib[c];
    }
    const double scale = (double)prod * a.norm_const;
    const bool usable = valid && key >= 0;
    long long k = usable ? key : 0;
    const int c2 = (int)(k % nc2); k /= nc2;
    const int c1 = (int)(k % nc1);
    const long long pil = k; k /= nc1;
    const int c0 = (int)(k % nc0);
    for (int o = sub; o < 9; o += G) {
        int first = 0, len = 0;
        if (usable) {
            const int cmin = c2 > 0 ? c2 - 1 : 0, cmax = c2 + 1 < nc2 ? c2 + 1 : nc2 - 1;
            const int dx = o / 3 - 1, dy = o % 3 - 1;
            const int x = c0 + dx, y = c1 + dy;
            if (x >= 0 && x < nc0 && y >= 0 && y < nc1)
                grid_pillar_range(a.grid, pil + (long long)dx * nc1 + dy, nc2, cmin, cmax, first, len);
        }
        ranges[wib][grp][o] = make_int2(first, len);
    }
    // (a wavefront's own LDS writes are in order with its reads: no barrier between the lanes of a group)
    const unsigned long long group_bits = (G == 64) ? ~0ull : (((1ull << (G & 63)) - 1ull) << (grp * G));
    const unsigned long long below = group_bits & pccnn_lanemask_lt();

    // walk(raw, cap): raw == 0 sums every hit, else only the capped subset; returns the hits of the point
    auto walk = [&](bool go, long long raw, long long cap, double &sum) -> int {
        int cnt = 0, r = 0, j0 = 0;
        int2 cur = ranges[wib][grp][0];
        bool active = go;
        sum = 0.0;
        while (__any(active)) {
            bool hit = false;
            float px = 0.f, py = 0.f, pz = 0.f;
            if (active) {
                const int j = j0 + sub;
                if (j < cur.y) {
                    const int64_t idx = cur.x + j;
                    px = a.pts[idx * 3 + 0];
                    py = a.pts[idx * 3 + 1];
                    pz = a.pts[idx * 3 + 2];
                    const float vx = (sx - px) * ir[0];
                    const float vy = (sy - py) * ir[1];
                    const float vz = (sz - pz) * ir[2];
                    const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                    hit = acc < 1.0f;
                }
            }
            const unsigned long long hits = __ballot(hit);
            if (active) {
                if (hit) {
                    bool take = true;
                    if (raw > 0) {
                        const long long rank = cnt + __popcll(hits & below);
                        take = (rank + 1) * cap / raw > rank * cap / raw;
                    }
                    if (take) {
                        const float d0 = (px - sx) * ib[0];
                        const float d1 = (py - sy) * ib[1];
                        const float d2 = (pz - sz) * ib[2];
                        const float dot = ((0.0f + d0 * d0) + d1 * d1) + d2 * d2;
                        sum += scale * (double)expf(dot * (-0.5f));
                    }
                }
                cnt += __popcll(hits & group_bits);
                j0 += G;
                if (j0 >= cur.y) {
                    j0 = 0;
                    if (++r < 9) cur = ranges[wib][grp][r];
                    else active = false;
                }
            }
        }
        return cnt;
    };
    double sum;
    const int cnt = walk(usable, 0, 0, sum);
    const bool redo = a.max_neighbors > 0 && cnt > a.max_neighbors;
    if (__any(redo)) {
        double capped_sum;
        (void)walk(redo, cnt, a.max_neighbors, capped_sum);
        if (redo) sum = capped_sum;
    }
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if (valid && sub == 0) {
        const int64_t at = a.order ? (int64_t)a.order[i] : i;
        const float v = (float)sum;
        a.out[at] = v;
        if (a.out_norm) {
            const long long cells = (long long)nc0 * nc1 * nc2;
            const int count = usable ? pdf_grid_cloud_count(a, key / cells, cells) : 1;
            a.out_norm[at] = __fdiv_rn(v, (float)count);
        }
    }
}

extern "C" int pccnn_compute_pdf_grid(int manifold_dims, const float *bandwidth, const float *pts_sorted,
                                      const int64_t *sorted_keys, int64_t n, const int32_t *sample_order,
                                      const int32_t *grid_ds, int64_t num_pillars, const int32_t *cell_table,
                                      int64_t total_cells, const int32_t *num_cells, const float *radii, int d,
                                      int max_neighbors, float *pdf_out, float *pdf_norm_out, void *stream)
{
    PCCNN_REQUIRE(d == 3, PCCNN_ERR_UNSUPPORTED, "pccnn_compute_pdf_grid: d=%d is not supported (3 only; use "
                  "pccnn_find_neighbors_* and pccnn_compute_pdf)", d);
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31) && num_pillars >= 0 && max_neighbors >= 0, PCCNN_ERR_INVALID,
                  "pccnn_compute_pdf_grid: n=%lld num_pillars=%lld max_neighbors=%d", (long long)n,
                  (long long)num_pillars, max_neighbors);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(bandwidth && pts_sorted && sorted_keys && grid_ds && num_cells && radii && pdf_out, PCCNN_ERR_INVALID,
                  "pccnn_compute_pdf_grid: null pointer");
    PCCNN_REQUIRE(!cell_table || (total_cells > 0 && total_cells < (1ll << 40)), PCCNN_ERR_INVALID,
                  "pccnn_compute_pdf_grid: total_cells=%lld", (long long)total_cells);
    PdfGridArgs a;
    a.pts = pts_sorted; a.keys = sorted_keys; a.order = sample_order;
    a.grid.cell_table = cell_table; a.grid.total_cells = total_cells; a.grid.grid_ds = grid_ds;
    a.grid.num_pillars = num_pillars; a.grid.pt_keys = sorted_keys; a.grid.n = n;
    a.num_cells = num_cells; a.radii = radii; a.bandwidth = bandwidth;
    a.norm_const = 1.0 / pow(2.0 * 3.1415, (double)(float)manifold_dims / 2.0);
    a.max_neighbors = max_neighbors; a.out = pdf_out; a.out_norm = pdf_norm_out; a.n = n;
    hipStream_t s = (hipStream_t)stream;
    {
        PccnnTimed timed(PCCNN_T_PDF, s);
        // one point per lane, unless that leaves the chip short of wavefronts: then 8 or 4 lanes per point, as long
        // as the launch still is one round of wavefronts (256 CUs x 32 x 64 lanes)
        const int64_t chip_lanes = 256 * 32 * 64;
        if (n * 8 <= chip_lanes) pdf_grid_group_kernel<8><<<pccnn_xcd_grid(pccnn_ceil_div(n * 8, 256), PDF_XCD_CHUNK), 256, 0, s>>>(a);
        else if (n * 4 <= chip_lanes) pdf_grid_group_kernel<4><<<pccnn_xcd_grid(pccnn_ceil_div(n * 4, 256), PDF_XCD_CHUNK), 256, 0, s>>>(a);
        else pdf_grid_kernel<<<pccnn_xcd_grid(pccnn_ceil_div(n, 256), PDF_XCD_CHUNK), 256, 0, s>>>(a);
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
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
