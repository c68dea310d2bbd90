/*
 * CPU oracle for the point-cloud operator path of pccnn_lib.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain scalar C, the
 * arithmetic the reference performs in its CUDA kernels and ATen call
 * sequences, so that the HIP kernels of this repository can be checked
 * against it.  It is never linked into, imported by or called from the
 * product library; only tests/, the smoke check and the benchmark's CPU
 * baseline leg use it.
 *
 * Every function cites the reference file:line it follows (paths relative
 * to the reference repository root).  Compile with contraction disabled
 * (-ffp-contract=off) so that fp32 expressions round exactly as written.
 *
 * PARITY UNPINNED: one piece only.  When a sample has more neighbors than
 * max_neighbors, orc_store_neighbors keeps an evenly spaced subset; the
 * reference keeps a random one seeded with time(NULL)
 * (pccnn_lib_ops/find_neighbors/store_neighbors.cu:66-99, find_neighbors.cu),
 * so which members survive cannot be compared, only the contract of its unit
 * test (count == cap, every member a distinct true neighbor).  Every other
 * function is pinned in tests/ by the formulas of the reference's own unit
 * tests, brute force, closed forms or hand-worked cases (the Poisson-disk
 * colour order and bit-to-dimension mapping: tests/golden/poisson_known_answers.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_D 6

/* fp32 reciprocal as torch::reciprocal computes it on a float tensor
 * (pccnn_lib_ops/compute_keys/compute_keys.cu:114,
 *  pccnn_lib_ops/find_neighbors/find_neighbors.cu:59,
 *  pccnn_lib_ops/compute_pdf/compute_pdf.cu:190). */
static inline float orc_rcp(float x) { return 1.0f / x; }

/* ------------------------------------------------------------------ keys */

/* pccnn_lib_ops/shared/grid_utils.cuh:57-68 (cell of a point) and :79-94
 * (row-major key with the batch id as the most significant digit), driven by
 * pccnn_lib_ops/compute_keys/compute_keys.cu:58-72. */
int orc_compute_keys(const float *pts, const int32_t *batch_ids,
                     const float *aabb_min, const int32_t *num_cells,
                     const float *cell_size, int64_t n, int d,
                     int64_t *keys_out)
{
    if (d < 2 || d > ORC_MAX_D) return -1;
    float inv[ORC_MAX_D];
    for (int i = 0; i < d; ++i) inv[i] = orc_rcp(cell_size[i]);
    for (int64_t p = 0; p < n; ++p) {
        int b = batch_ids[p];
        int cell[ORC_MAX_D];
        for (int i = 0; i < d; ++i) {
            float rel = (pts[p * d + i] - aabb_min[(int64_t)b * d + i]) * inv[i];
            int c = (int)floorf(rel);
            if (c < 0) c = 0;
            if (c > num_cells[i] - 1) c = num_cells[i] - 1;
            cell[i] = c;
        }
        int64_t key = 0, accum = 1;
        for (int i = d - 1; i >= 0; --i) {
            key += (int64_t)cell[i] * accum;
            accum *= num_cells[i];
        }
        keys_out[p] = key + accum * (int64_t)b;
    }
    return 0;
}

/* Stable argsort of the keys: what pccnn_lib/pc/Grid.py:52 asks of
 * torch.argsort, with ties resolved in original-index order (the reference
 * leaves tie order unspecified; stable order is this build's choice). */
typedef struct { int64_t key; int32_t idx; } orc_kv;
static int orc_kv_cmp(const void *a, const void *b)
{
    const orc_kv *x = (const orc_kv *)a, *y = (const orc_kv *)b;
    if (x->key < y->key) return -1;
    if (x->key > y->key) return 1;
    return (x->idx > y->idx) - (x->idx < y->idx);
}
int orc_argsort_keys(const int64_t *keys, int64_t n, int32_t *perm_out)
{
    orc_kv *kv = (orc_kv *)malloc(sizeof(orc_kv) * (size_t)(n > 0 ? n : 1));
    if (!kv) return -1;
    for (int64_t i = 0; i < n; ++i) { kv[i].key = keys[i]; kv[i].idx = (int32_t)i; }
    qsort(kv, (size_t)n, sizeof(orc_kv), orc_kv_cmp);
    for (int64_t i = 0; i < n; ++i) perm_out[i] = kv[i].idx;
    free(kv);
    return 0;
}

/* ------------------------------------------------------------------ grid */

/* pccnn_lib_ops/shared/grid_utils.cuh:128-137: index of the (batch, c0, c1)
 * pillar a key falls in = key / prod(num_cells[2:]). */
static inline int64_t orc_pillar_of_key(int64_t key, const int32_t *nc, int d)
{
    int64_t div = 1;
    for (int i = 2; i < d; ++i) div *= nc[i];
    return key / div;
}

/* pccnn_lib_ops/build_grid/build_grid_ds.cu:44-67: (first, last+1) index of
 * each pillar's run in the sorted key array; untouched pillars stay (0,0). */
int orc_build_grid_ds(const int64_t *sorted_keys, int64_t n,
                      const int32_t *num_cells, int d, int64_t table_pillars,
                      int32_t *ds_out /* [table_pillars][2], zero-filled here */)
{
    memset(ds_out, 0, sizeof(int32_t) * 2 * (size_t)table_pillars);
    for (int64_t i = 0; i < n; ++i) {
        int64_t ds = orc_pillar_of_key(sorted_keys[i], num_cells, d);
        if (ds < 0 || ds >= table_pillars) return -2;
        if (i - 1 >= 0 && ds != orc_pillar_of_key(sorted_keys[i - 1], num_cells, d))
            ds_out[2 * ds] = (int32_t)i;
        if (i + 1 == n)
            ds_out[2 * ds + 1] = (int32_t)n;
        else if (ds != orc_pillar_of_key(sorted_keys[i + 1], num_cells, d))
            ds_out[2 * ds + 1] = (int32_t)(i + 1);
    }
    return 0;
}

/* ------------------------------------------------------------- neighbors */

/* pccnn_lib_ops/find_neighbors/find_ranges_grid_ds.cu:306-338: the offset
 * table.  Offsets run over {-1,0,1} in dims 0..max(D-2,1); the last dim is
 * forced to 0 unless D == 2.  Returns the number of offsets. */
int orc_offsets(int d, int32_t *out /* [3^max(D-1,2)][d] */)
{
    int cells = 3, n_off = 3;
    int top = (d - 2 > 1) ? d - 2 : 1;
    for (int i = 0; i < top; ++i) n_off *= cells;
    for (int i = 0; i < n_off; ++i) {
        int aux = i;
        int cur[ORC_MAX_D] = {0};
        for (int j = top; j >= 0; --j) { cur[j] = aux % cells - 1; aux /= cells; }
        if (d != 2) cur[d - 1] = 0;
        for (int j = 0; j < d; ++j) out[i * d + j] = cur[j];
    }
    return n_off;
}

/* pccnn_lib_ops/find_neighbors/find_ranges_grid_ds.cu:65-165 (D > 2) and
 * :203-236 (D == 2).  The reference's interleaved binary searches return the
 * index range of keys in [minKey, maxKey] inside the pillar, or (0,0) when
 * there is none; that is what is computed here with plain bound searches. */
int orc_find_ranges(const int64_t *sample_keys, int64_t m,
                    const int64_t *pt_keys, int64_t n,
                    const int32_t *grid_ds, const int32_t *num_cells, int d,
                    int32_t *ranges_out /* [m][n_off][2] */)
{
    int32_t offs[243 * ORC_MAX_D];
    int n_off = orc_offsets(d, offs);
    int64_t total_cells = 1;
    for (int i = 0; i < d; ++i) total_cells *= num_cells[i];
    (void)n;
    memset(ranges_out, 0, sizeof(int32_t) * 2 * (size_t)m * (size_t)n_off);
    for (int64_t s = 0; s < m; ++s) {
        /* grid_utils.cuh:104-118: key -> (batch, c0..cD-1) */
        int64_t aux = sample_keys[s];
        int cell0[ORC_MAX_D + 1];
        for (int i = d - 1; i >= 0; --i) { cell0[i + 1] = (int)(aux % num_cells[i]); aux /= num_cells[i]; }
        cell0[0] = (int)aux;
        for (int o = 0; o < n_off; ++o) {
            int cell[ORC_MAX_D + 1];
            cell[0] = cell0[0];
            for (int i = 0; i < d; ++i) cell[i + 1] = cell0[i + 1] + offs[o * d + i];
            int inside = 1;
            int chk = (d == 2) ? d : d - 1;
            for (int i = 0; i < chk; ++i)
                inside = inside && cell[i + 1] >= 0 && cell[i + 1] < num_cells[i];
            if (!inside) continue;
            /* grid_utils.cuh:148-153 */
            int64_t ds_idx = (int64_t)cell[0] * num_cells[0] * num_cells[1]
                           + (int64_t)cell[1] * num_cells[1] + cell[2];
            int32_t lo = grid_ds[2 * ds_idx], hi = grid_ds[2 * ds_idx + 1];
            int32_t *out = ranges_out + 2 * (s * n_off + o);
            if (d == 2) { out[0] = lo; out[1] = hi; continue; }
            if (hi - lo - 1 < 0) continue;
            int64_t key = 0, accum = 1;
            for (int i = d - 1; i >= 0; --i) { key += (int64_t)cell[i + 1] * accum; accum *= num_cells[i]; }
            key += accum * (int64_t)cell[0];
            int64_t max_key = key + 1, min_key = key - 1;
            if (key / total_cells != max_key / total_cells)
                max_key = (key / total_cells) * total_cells + total_cells - 1;
            if (key / total_cells != min_key / total_cells)
                min_key = (key / total_cells) * total_cells;
            int32_t a = lo, b = hi;           /* first index with key >= min_key */
            while (a < b) { int32_t mid = a + (b - a) / 2; if (pt_keys[mid] < min_key) a = mid + 1; else b = mid; }
            int32_t first = a;
            a = lo; b = hi;                    /* first index with key > max_key */
            while (a < b) { int32_t mid = a + (b - a) / 2; if (pt_keys[mid] <= max_key) a = mid + 1; else b = mid; }
            int32_t last = a;
            if (last > first) { out[0] = first; out[1] = last; }
        }
    }
    return n_off;
}

/* pccnn_lib_ops/find_neighbors/count_neighbors.cu:77-91 and
 * store_neighbors.cu:160-172: fp32, diff = sample - point, times the fp32
 * reciprocal radius, dot accumulated d = 0..D-1 from 0
 * (shared/math_helper.cuh:306-321), sqrt, strict < 1. */
static inline int orc_is_neighbor(const float *s, const float *p, const float *inv_r, int d)
{
    float acc = 0.0f;
    for (int i = 0; i < d; ++i) {
        float v = (s[i] - p[i]) * inv_r[i];
        acc = acc + v * v;
    }
    return sqrtf(acc) < 1.0f;
}

/* Count pass (count_neighbors.cu:38-104). */
int orc_count_neighbors(const float *samples, int64_t m, const float *pts_sorted,
                        const int32_t *ranges, int n_off, const float *radii, int d,
                        int32_t *counts_out)
{
    float inv[ORC_MAX_D];
    for (int i = 0; i < d; ++i) inv[i] = orc_rcp(radii[i]);
    for (int64_t s = 0; s < m; ++s) {
        int32_t c = 0;
        for (int o = 0; o < n_off; ++o) {
            const int32_t *r = ranges + 2 * (s * n_off + o);
            for (int32_t j = r[0]; j < r[1]; ++j)
                c += orc_is_neighbor(samples + s * d, pts_sorted + (int64_t)j * d, inv, d);
        }
        counts_out[s] = c;
    }
    return 0;
}

/* Store pass (store_neighbors.cu:129-175, 253-279): pairs (sorted point
 * index, sample index) grouped by sample; `ends` is the inclusive running
 * total.  The reference's order inside a sample is whatever its atomics give;
 * here it is ascending range, ascending index.  With max_neighbors > 0
 * (store_neighbors.cu:46-113, 219-251) counts are clamped; when a sample has
 * more hits than the cap the reference keeps a time-seeded random subset, which
 * nothing can pin -- this restatement keeps hit r (0-based, in the order above)
 * iff floor((r+1)*cap/cnt) > floor(r*cap/cnt): `cap` hits spread evenly. */
int64_t orc_store_neighbors(const float *samples, int64_t m, const float *pts_sorted,
                            const int32_t *ranges, int n_off, const float *radii, int d,
                            const int32_t *counts, int32_t max_neighbors,
                            int32_t *neigh_out /* [T][2] or NULL */, int32_t *ends_out)
{
    float inv[ORC_MAX_D];
    for (int i = 0; i < d; ++i) inv[i] = orc_rcp(radii[i]);
    int64_t total = 0;
    for (int64_t s = 0; s < m; ++s) {
        int32_t cnt = counts[s];
        int32_t keep = (max_neighbors > 0 && cnt > max_neighbors) ? max_neighbors : cnt;
        if (neigh_out) {
            int64_t r = 0;
            for (int o = 0; o < n_off; ++o) {
                const int32_t *rg = ranges + 2 * (s * n_off + o);
                for (int32_t j = rg[0]; j < rg[1]; ++j) {
                    if (!orc_is_neighbor(samples + s * d, pts_sorted + (int64_t)j * d, inv, d)) continue;
                    int64_t slot = r;
                    int take = 1;
                    if (keep != cnt) {
                        slot = (r * keep) / cnt;
                        take = ((r + 1) * keep) / cnt > slot;
                    }
                    if (take) {
                        neigh_out[2 * (total + slot)] = j;
                        neigh_out[2 * (total + slot) + 1] = (int32_t)s;
                    }
                    ++r;
                }
            }
        }
        total += keep;
        ends_out[s] = (int32_t)total;
    }
    return total;
}

/* O(N*M) search with the same predicate, restricted to equal batch ids:
 * the formulation of unit_test/test_find_neighs.py:57-67 with the kernel's
 * predicate.  Counts only when neigh_out is NULL. */
int64_t orc_brute_force_neighbors(const float *samples, const int32_t *sample_batch, int64_t m,
                                  const float *pts, const int32_t *pt_batch, int64_t n,
                                  const float *radii, int d,
                                  int32_t *neigh_out, int32_t *ends_out)
{
    float inv[ORC_MAX_D];
    for (int i = 0; i < d; ++i) inv[i] = orc_rcp(radii[i]);
    int64_t total = 0;
    for (int64_t s = 0; s < m; ++s) {
        for (int64_t j = 0; j < n; ++j) {
            if (pt_batch[j] != sample_batch[s]) continue;
            if (!orc_is_neighbor(samples + s * d, pts + j * d, inv, d)) continue;
            if (neigh_out) { neigh_out[2 * total] = (int32_t)j; neigh_out[2 * total + 1] = (int32_t)s; }
            ++total;
        }
        ends_out[s] = (int32_t)total;
    }
    return total;
}

/* ------------------------------------------------------------------- pdf */

/* pccnn_lib_ops/compute_pdf/compute_pdf.cu:42-76.  Per pair the product
 * (prod inv_bw) * (1/pow(2*3.1415, m/2)) * exp(...) is formed in double
 * (the middle factor is a double literal expression) and added to an fp32
 * accumulator, i.e. accum = (float)((double)accum + term). */
int orc_compute_pdf(int manifold_dims, const float *bandwidth, const float *pts, int64_t n, int d,
                    const int32_t *neigh, const int32_t *ends, float *pdf_out)
{
    float ib[ORC_MAX_D];
    for (int i = 0; i < d; ++i) ib[i] = orc_rcp(bandwidth[i]);
    float mdims = (float)manifold_dims;
    for (int64_t s = 0; s < n; ++s) {
        int32_t lo = s > 0 ? ends[s - 1] : 0, hi = ends[s];
        float accum = 0.0f;
        for (int32_t t = lo; t < hi; ++t) {
            int32_t j = neigh[2 * t];
            float dot = 0.0f;
            for (int i = 0; i < d; ++i) {
                float v = (pts[(int64_t)j * d + i] - pts[s * d + i]) * ib[i];
                dot = dot + v * v;
            }
            float e = expf(dot * (-0.5f));
            float local = 1.0f;
            for (int i = 0; i < d; ++i) local *= ib[i];
            accum = (float)((double)accum + (double)local * (1.0 / pow(2.0 * 3.1415, mdims / 2.0)) * (double)e);
        }
        pdf_out[s] = accum;
    }
    return 0;
}

/* pccnn_lib_ops/compute_pdf/compute_pdf.cu:100-148: gradient of
 * sum_s g_s * pdf_s w.r.t. the points (self accumulates +, neighbor gets -). */
int orc_compute_pdf_grads(int manifold_dims, const float *bandwidth, const float *pts, int64_t n, int d,
                          const int32_t *neigh, const int32_t *ends, const float *in_grads,
                          float *pt_grads_out /* [n][d], zero-filled here */)
{
    float ib[ORC_MAX_D];
    for (int i = 0; i < d; ++i) ib[i] = orc_rcp(bandwidth[i]);
    float mdims = (float)manifold_dims;
    double *acc = (double *)calloc((size_t)(n * d > 0 ? n * d : 1), sizeof(double));
    if (!acc) return -1;
    for (int64_t s = 0; s < n; ++s) {
        int32_t lo = s > 0 ? ends[s - 1] : 0, hi = ends[s];
        float g = in_grads[s];
        for (int32_t t = lo; t < hi; ++t) {
            int32_t j = neigh[2 * t];
            float diff[ORC_MAX_D];
            float dot = 0.0f;
            for (int i = 0; i < d; ++i) {
                diff[i] = (pts[(int64_t)j * d + i] - pts[s * d + i]) * ib[i];
                dot = dot + diff[i] * diff[i];
            }
            float e = expf(dot * (-0.5f));
            float local = 1.0f;
            for (int i = 0; i < d; ++i) local *= ib[i];
            local = (float)((double)local * (1.0 / pow(2.0 * 3.1415, mdims / 2.0)) * (double)e);
            for (int i = 0; i < d; ++i) {
                float lg = diff[i] * ib[i] * g * local;
                acc[s * d + i] += lg;
                acc[(int64_t)j * d + i] -= lg;
            }
        }
    }
    for (int64_t i = 0; i < n * d; ++i) pt_grads_out[i] = (float)acc[i];
    free(acc);
    return 0;
}

/* --------------------------------------------------------------- pooling */

/* pccnn_lib_ops/poisson_disk_sampling/poisson_disk_sampling.cu:56-105 and
 * :116-195.  All arrays are in sorted-index space.  2^D passes, pass c keeps
 * cells whose index parity in dim i equals bit i of c; inside a pass cells do
 * not interact, inside a cell points are visited in sorted order, and a point
 * is selected iff none of its listed neighbors is selected yet. */
int64_t orc_poisson_disk(const int64_t *sorted_keys, int64_t n,
                         const int32_t *neigh, const int32_t *ends,
                         const int32_t *num_cells, int d,
                         int32_t *used_out /* [n] */)
{
    memset(used_out, 0, sizeof(int32_t) * (size_t)n);
    int calls = 1 << d;
    for (int c = 0; c < calls; ++c) {
        for (int64_t i = 0; i < n; ++i) {
            int64_t aux = sorted_keys[i];
            int ok = 1;
            for (int k = d - 1; k >= 0; --k) {
                int ck = (int)(aux % num_cells[k]);
                aux /= num_cells[k];
                ok = ok && ((ck % 2) == ((c >> k) & 1));
            }
            if (!ok) continue;
            int32_t lo = i > 0 ? ends[i - 1] : 0, hi = ends[i];
            int valid = 1;
            for (int32_t t = lo; t < hi; ++t) valid = valid && (used_out[neigh[2 * t]] == 0);
            if (valid) used_out[i] = 1;
        }
    }
    int64_t cnt = 0;
    for (int64_t i = 0; i < n; ++i) cnt += used_out[i];
    return cnt;
}

/* ------------------------------------------------------------------ conv */

/* Per-pair basis values, fp32 like the ATen sequences they restate.
 *
 * kind 0 (KPConv): pccnn_lib_ops/pcconvs/shared/pt_diff.cu:35-45 then
 *   kernel_pts_basis.cu:30-38:  d = (pts[n]-samples[s]) * (1/r);
 *   w_k = clamp(1 - sqrt(max(sum_i (kp_ki - d_i)^2, 0)) / sigma, 0, 1).
 * kind 1 (MCConv): pt_diff as above, pccnn_lib_ops/pcconvs/mcconv.cu:52-53
 *   (pdf gathered by neighbor) and mlp_basis.cu:35-47:
 *   w_h = leaky_relu(sum_i d_i * A_ih + b_h, 0.2) / pdf[n].
 * basis_out is [T][K].  diff_out (optional) is [T][D]. */
int orc_conv_basis(int kind, const float *pts, const float *samples, const int32_t *neigh, int64_t t_pairs,
                   const float *radii, int d, int k_basis,
                   const float *kp_or_axis, const float *bias, float sigma, const float *pdf,
                   float *basis_out, float *diff_out)
{
    float inv[ORC_MAX_D];
    for (int i = 0; i < d; ++i) inv[i] = orc_rcp(radii[i]);
    for (int64_t t = 0; t < t_pairs; ++t) {
        int32_t nidx = neigh[2 * t], sidx = neigh[2 * t + 1];
        float diff[ORC_MAX_D];
        for (int i = 0; i < d; ++i) {
            diff[i] = (pts[(int64_t)nidx * d + i] - samples[(int64_t)sidx * d + i]) * inv[i];
            if (diff_out) diff_out[t * d + i] = diff[i];
        }
        for (int k = 0; k < k_basis; ++k) {
            float w;
            if (kind == 0) {
                float acc = 0.0f;
                for (int i = 0; i < d; ++i) {
                    float v = kp_or_axis[k * d + i] - diff[i];
                    acc = acc + v * v;
                }
                if (acc < 0.0f) acc = 0.0f;
                float r = 1.0f - sqrtf(acc) / sigma;
                w = r < 0.0f ? 0.0f : (r > 1.0f ? 1.0f : r);
            } else {
                float acc = 0.0f;
                for (int i = 0; i < d; ++i) acc = acc + diff[i] * kp_or_axis[i * k_basis + k];
                acc = acc + bias[k];
                acc = acc > 0.0f ? acc : acc * 0.2f;
                w = acc / pdf[nidx];
            }
            basis_out[t * k_basis + k] = w;
        }
    }
    return 0;
}

/* pccnn_lib_ops/pcconvs/shared/feat_basis_proj.cu:56-128:
 * P[s][f][k] = sum over the pairs t of sample s of F[n_t][f] * w[t][k]
 * (k fastest).  Accumulated in double, rounded once. */
int orc_feat_basis_proj(const float *basis, const float *feats, const int32_t *neigh, const int32_t *ends,
                        int64_t m, int c_in, int k_basis, float *proj_out)
{
    double *acc = (double *)malloc(sizeof(double) * (size_t)c_in * (size_t)k_basis);
    if (!acc) return -1;
    for (int64_t s = 0; s < m; ++s) {
        int32_t lo = s > 0 ? ends[s - 1] : 0, hi = ends[s];
        for (int i = 0; i < c_in * k_basis; ++i) acc[i] = 0.0;
        for (int32_t t = lo; t < hi; ++t) {
            const float *f = feats + (int64_t)neigh[2 * t] * c_in;
            const float *w = basis + (int64_t)t * k_basis;
            for (int a = 0; a < c_in; ++a)
                for (int k = 0; k < k_basis; ++k) acc[a * k_basis + k] += (double)f[a] * (double)w[k];
        }
        for (int i = 0; i < c_in * k_basis; ++i) proj_out[s * c_in * k_basis + i] = (float)acc[i];
    }
    free(acc);
    return 0;
}

/* pccnn_lib_ops/pcconvs/shared/feat_basis_proj_grads.cu:62-153:
 * dF[n_t][f] += sum_k dP[s][f][k] * w[t][k];  dw[t][k] = sum_f dP[s][f][k] * F[n_t][f]. */
int orc_feat_basis_proj_grads(const float *basis, const float *feats, const int32_t *neigh, const int32_t *ends,
                              int64_t m, int64_t n, int c_in, int k_basis, const float *proj_grads,
                              float *feat_grads_out /* [n][c_in] */, float *basis_grads_out /* [T][k] */)
{
    double *facc = (double *)calloc((size_t)(n * c_in > 0 ? n * c_in : 1), sizeof(double));
    if (!facc) return -1;
    for (int64_t s = 0; s < m; ++s) {
        int32_t lo = s > 0 ? ends[s - 1] : 0, hi = ends[s];
        const float *dp = proj_grads + s * c_in * k_basis;
        for (int32_t t = lo; t < hi; ++t) {
            int32_t nidx = neigh[2 * t];
            const float *f = feats + (int64_t)nidx * c_in;
            const float *w = basis + (int64_t)t * k_basis;
            for (int k = 0; k < k_basis; ++k) {
                double a = 0.0;
                for (int c = 0; c < c_in; ++c) a += (double)dp[c * k_basis + k] * (double)f[c];
                basis_grads_out[(int64_t)t * k_basis + k] = (float)a;
            }
            for (int c = 0; c < c_in; ++c) {
                double a = 0.0;
                for (int k = 0; k < k_basis; ++k) a += (double)dp[c * k_basis + k] * (double)w[k];
                facc[(int64_t)nidx * c_in + c] += a;
            }
        }
    }
    for (int64_t i = 0; i < n * c_in; ++i) feat_grads_out[i] = (float)facc[i];
    free(facc);
    return 0;
}

/* pccnn_lib_ops/pcconvs/shared/compute_variance_weights.cu:38-108 with pDivideNumNeighs = false (the KPConv
 * and MCConv callers, kpconv.cu:133-135, mcconv.cu:169-171): per sample the double sum over ordered pairs
 * (i, j) of its neighbors of (w_i . w_j) * (F_i . F_j); then :168-169, the reciprocal of the mean over the
 * samples.  Written as the literal O(n^2) loops, accumulated in double.  per_sample_out may be NULL. */
double orc_variance_weights(const float *basis, const float *feats, const int32_t *neigh, const int32_t *ends,
                            int64_t m, int c_in, int k_basis, double *per_sample_out)
{
    double total = 0.0;
    for (int64_t s = 0; s < m; ++s) {
        int32_t lo = s > 0 ? ends[s - 1] : 0, hi = ends[s];
        double acc = 0.0;
        for (int32_t i = lo; i < hi; ++i) {
            const float *wi = basis + (int64_t)i * k_basis;
            const float *fi = feats + (int64_t)neigh[2 * i] * c_in;
            for (int32_t j = lo; j < hi; ++j) {
                const float *wj = basis + (int64_t)j * k_basis;
                const float *fj = feats + (int64_t)neigh[2 * j] * c_in;
                double sw = 0.0, sf = 0.0;
                for (int k = 0; k < k_basis; ++k) sw += (double)wi[k] * (double)wj[k];
                for (int c = 0; c < c_in; ++c) sf += (double)fi[c] * (double)fj[c];
                acc += sw * sf;
            }
        }
        if (per_sample_out) per_sample_out[s] = acc;
        total += acc;
    }
    return 1.0 / (total / (double)m);
}
