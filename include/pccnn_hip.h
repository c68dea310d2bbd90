/*
 * pccnn_hip.h -- C ABI of libpccnn_hip.so: the point-cloud operator path of
 * pccnn_lib (cell keys, key sort, pillar grid, radius neighbor search, Gaussian
 * KDE, Poisson-disk selection, KPConv / MCConv forward and backward) as
 * hand-written HIP kernels for gfx950 (MI355X, CDNA4, wave64).
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless its name starts with `h_`.
 *  - Tensors are dense, row-major, of exactly the stated element type.
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).  All
 *    work is enqueued on it.  The operator entry points neither synchronise
 *    nor allocate: temporary storage comes in through `workspace` arguments
 *    whose minimum size the matching *_workspace_bytes function reports.
 *    Three groups are the exception, and each says so where it is declared:
 *    the "host sequences" (they end with a read-back: the synchronous ones
 *    wait for `stream` with hipStreamSynchronize, and every one keeps a small
 *    page-locked staging block per host thread, allocated with hipHostMalloc
 *    on first use and kept until the process ends); pccnn_sort_keys_static
 *    (its storage is a static device array); and the optional timing hooks
 *    (pccnn_timing_*: they create events while switched on).
 *  - Return value: 0 on success, a negative PCCNN_ERR_* code otherwise;
 *    pccnn_last_error() then returns a thread-local description.  Arguments
 *    are validated on the host before any kernel is launched.
 *  - D (point dimensionality) is 2 to 6; the measured
 *    kernels are the 3-dimensional ones, other D run slower general forms.
 *    An entry point that is 3-dimensional only says so and returns
 *    PCCNN_ERR_UNSUPPORTED for another D.
 *
 * Each entry point cites the reference interface it replaces (paths relative
 * to the reference repository; *.cuh lines are the host-function prototypes
 * that pccnn_lib_ops/ops_list.cpp:26-54 exports to Python).
 */
#ifndef PCCNN_HIP_H
#define PCCNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCCNN_OK 0
#define PCCNN_ERR_INVALID (-1)     /* null pointer, negative size, inconsistent shapes */
#define PCCNN_ERR_UNSUPPORTED (-2) /* valid request this build has no kernel for */
#define PCCNN_ERR_WORKSPACE (-3)   /* workspace missing or too small */
#define PCCNN_ERR_HIP (-4)         /* a HIP runtime call or kernel launch failed */

const char *pccnn_last_error(void);
int pccnn_version(void);

/* ---- bounding box -------------------------------------------------------
 * Replaces pccnn_lib/pc/BoundingBox.py:17-18 (torch_scatter scatter_min /
 * scatter_max followed by -1e-6 / +1e-6 in fp32).
 * pts f32[n,d], batch_ids i32[n] in [0,batch_size) -> aabb_min/max f32[batch_size,d]. */
int pccnn_bounding_box(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                       float *aabb_min_out, float *aabb_max_out, void *stream);
/* Grid size for a cell size: replaces the torch arithmetic of pccnn_lib/pc/Grid.py:26-28,
 * num_cells[k] = max over the clouds of int32((aabb_max - aabb_min) / cell_size) + 1 (fp32 division, truncation).
 * aabb_min/max f32[batch_size,d], cell_size f32[d] -> num_cells_out i32[d]. */
int pccnn_num_cells(const float *aabb_min, const float *aabb_max, const float *cell_size, int batch_size, int d,
                    int32_t *num_cells_out, void *stream);

/* ---- cell keys ----------------------------------------------------------
 * Replaces compute_keys (pccnn_lib_ops/compute_keys/compute_keys.cuh:26-31,
 * compute_keys.cu:78-127).  num_cells i32[d] and cell_size f32[d] live on the
 * device like the tensors the reference receives.  keys_out i64[n]. */
int pccnn_compute_keys(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                       const int32_t *num_cells, const float *cell_size, int64_t n, int d,
                       int64_t *keys_out, void *stream);

/* ---- key sort -----------------------------------------------------------
 * Replaces torch.argsort(cell_ids) and the index_select gathers that follow it
 * (pccnn_lib/pc/Grid.py:52,68-70; pccnn_lib/pc/Neighborhood.py:27-32).
 * Stable LSD radix sort of the low `key_bits` bits of non-negative 64-bit keys
 * (key_bits <= 0 means 64).  Outputs: sorted_keys_out i64[n], perm_out i32[n]
 * (perm_out[i] = original index of the i-th smallest key, ties in original
 * order) and, when pts != NULL, sorted_pts_out f32[n,d] = pts[perm_out]. */
size_t pccnn_sort_keys_workspace_bytes(int64_t n);
int pccnn_sort_keys(const int64_t *keys, int64_t n, int key_bits, int64_t *sorted_keys_out, int32_t *perm_out,
                    const float *pts, int d, float *sorted_pts_out,
                    void *workspace, size_t workspace_bytes, void *stream);
/* pccnn_sort_keys without the workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments, same results; the temporary storage is an array built into the library's device image
 * (about 16 MiB per GPU, held until the process ends), so n is limited to PCCNN_SORT_KEYS_STATIC_MAX keys and a
 * larger n returns PCCNN_ERR_UNSUPPORTED.  The call allocates nothing, frees nothing and creates no events; the
 * device current at the call must be the stream's.  The first call on a device looks up the array's device
 * address (make it outside a capture).  Every call on a GPU uses that GPU's one array: calls that overlap on
 * one GPU (two streams, two threads) race; calls on one stream, or ordered by events, do not. */
#define PCCNN_SORT_KEYS_STATIC_MAX (1 << 20)
int pccnn_sort_keys_static(const int64_t *keys, int64_t n, int key_bits, int64_t *sorted_keys_out, int32_t *perm_out,
                           const float *pts, int d, float *sorted_pts_out, void *stream);

/* ---- pillar grid --------------------------------------------------------
 * Replaces build_grid_ds (pccnn_lib_ops/build_grid/build_grid_ds.cuh:25-28,
 * build_grid_ds.cu:72-114).  sorted_keys i64[n] ascending; grid_ds_out
 * i32[num_pillars,2] with num_pillars = batch_size*num_cells[0]*num_cells[1];
 * (first, last+1) of each pillar's run, (0,0) for empty pillars. */
int pccnn_build_grid_ds(const int64_t *sorted_keys, int64_t n, const int32_t *num_cells, int d,
                        int64_t num_pillars, int32_t *grid_ds_out, void *stream);

/* ---- radius neighbor search --------------------------------------------
 * Replaces find_neighbors (pccnn_lib_ops/find_neighbors/find_neighbors.cuh:33-41,
 * find_neighbors.cu:27-66) as two calls around the one size the host must learn:
 *
 *   pccnn_find_neighbors_count  -> ends_out i32[m]: inclusive running total of
 *       min(count, max_neighbors or inf) per sample (the `start ids` tensor the
 *       reference returns);  the caller copies ends_out[m-1] (= T) to the host,
 *       allocates neigh i32[T,2], then calls
 *   pccnn_find_neighbors_fill   -> neigh_out[t] = (point, sample).
 *
 * pts_sorted f32[n,d] / pt_keys_sorted i64[n]: points in key order;
 * samples f32[m,d] / sample_keys i64[m]: queries in any order, keyed on the
 * points' grid; grid_ds i32[num_pillars,2] from pccnn_build_grid_ds; radii f32[d] (device).
 * sample_order i32[m] (nullable): a permutation that lists the samples in
 * ascending key order -- tiles of consecutive entries then share their cell
 * walk; NULL means natural order.  samples_presorted != 0 (only with a sample_order): the arrays `samples`
 * and `sample_keys` are already listed in that order (entry i belongs to sample sample_order[i]), as
 * pccnn_sort_keys leaves them, so the kernels read them as contiguous runs instead of gathering.
 * max_neighbors 0 = unlimited; otherwise a
 * sample with more hits keeps max_neighbors of them, evenly spaced in its hit
 * order (the reference keeps a time-seeded random subset there).
 * point_remap i32[n] (nullable): when given, column 0 of neigh_out is
 * point_remap[sorted index] (fuses pccnn_lib/pc/Neighborhood.py:47-53), else the
 * sorted index as in the reference op.  Pairs are grouped by ascending sample
 * index; inside a sample they are in ascending sorted-point order.
 * Both calls take the same workspace of pccnn_find_neighbors_workspace_bytes(n, m) bytes, untouched in between and
 * with the same arguments: count leaves the per-sample raw counts in it and, for large uncapped searches, one bit
 * per candidate it tested (neighbor or not), from which fill writes the pairs without testing again; otherwise
 * fill packs the sorted points into 16-byte records there and repeats the walk.  The count call also
 * leaves the pair total T as an int64 in the first 8 bytes of the workspace: ends_out is 32-bit like the
 * reference's tensor and wraps beyond 2^31 - 1 pairs, that number does not, so a caller that reads it instead of
 * ends_out[m-1] can refuse such a search. */
size_t pccnn_find_neighbors_workspace_bytes(int64_t n, int64_t m);
/* Optional accelerator for the search (no counterpart in the reference, which binary-searches the sorted
 * keys inside each pillar, find_ranges_grid_ds.cu:111-163): cell_table_out i32[total_cells + 1], entry c =
 * index of the first sorted point with key >= c, total_cells = batch_size * prod(num_cells).  When passed to
 * the two calls below, the range of the three cells a pillar contributes is two table reads; with NULL the
 * pillar table and a binary search are used.  Same results either way. */
int pccnn_build_cell_table(const int64_t *sorted_keys, int64_t n, int64_t total_cells, int32_t *cell_table_out,
                           void *stream);
/* Keys, sort, pillar table and (cell_table_out non-NULL) cell table of one grid in one call: the work of
 * Grid.compute_cell_ids + Grid.build_ds (pccnn_lib/pc/Grid.py:40-72).  Arguments as for pccnn_compute_keys,
 * pccnn_sort_keys (key_bits, workspace of pccnn_grid_build_workspace_bytes(n) bytes), pccnn_build_grid_ds
 * (num_pillars) and pccnn_build_cell_table (total_cells); keys_out i64[n] are the unsorted keys. */
size_t pccnn_grid_build_workspace_bytes(int64_t n);
int pccnn_grid_build(const float *pts, const int32_t *batch_ids, const float *aabb_min, const int32_t *num_cells,
                     const float *cell_size, int64_t n, int d, int key_bits, int64_t num_pillars,
                     int64_t total_cells, int64_t *keys_out, int64_t *sorted_keys_out, int32_t *perm_out,
                     float *sorted_pts_out, int32_t *grid_ds_out, int32_t *cell_table_out, void *workspace,
                     size_t workspace_bytes, void *stream);
int pccnn_find_neighbors_count(const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                               const float *samples, const int64_t *sample_keys, int64_t m,
                               const int32_t *sample_order, int samples_presorted,
                               const int32_t *grid_ds, int64_t num_pillars,
                               const int32_t *cell_table, int64_t total_cells,
                               const int32_t *num_cells, const float *radii, int d, int max_neighbors,
                               int32_t *ends_out,
                               void *workspace, size_t workspace_bytes, void *stream);
int pccnn_find_neighbors_fill(const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                              const float *samples, const int64_t *sample_keys, int64_t m,
                              const int32_t *sample_order, int samples_presorted,
                              const int32_t *grid_ds, int64_t num_pillars,
                              const int32_t *cell_table, int64_t total_cells,
                              const int32_t *num_cells, const float *radii, int d, int max_neighbors,
                              const int32_t *ends,
                              const int32_t *point_remap, int64_t t, int32_t *neigh_out,
                              void *workspace, size_t workspace_bytes, void *stream);

/* ---- Gaussian KDE -------------------------------------------------------
 * Replaces compute_pdf / compute_pdf_grads (pccnn_lib_ops/compute_pdf/compute_pdf.cuh:28-51,
 * compute_pdf.cu:153-257).  neigh i32[t,2] = (point, sample) in original point
 * ids, ends i32[n]; samples are the points themselves.  pdf_out f32[n];
 * pt_grads_out f32[n,d].  Coordinates are gathered by original index, one
 * cache line per pair when the points are in no spatial order;
 * pccnn_compute_pdf_sorted and pccnn_compute_pdf_grid below work on the
 * grid's sorted copy and read whole lines.  pccnn_compute_pdf_grads adds
 * into pt_grads_out with float atomics (pccnn_lib_ops/compute_pdf/compute_pdf.cu:153-257
 * does the same), so its sums depend on the order of arrival in the last bit. */
int pccnn_compute_pdf(int manifold_dims, const float *bandwidth, const float *pts, int64_t n, int d,
                      const int32_t *neigh, int64_t t, const int32_t *ends, float *pdf_out, void *stream);
/* Same estimate for a pair list left in sorted-index space (pccnn_find_neighbors_fill without point_remap):
 * column 0 of neigh_sorted indexes pts_sorted, sample i is samples[i] (the cloud in its original order).  The
 * neighbors of a sample are then runs of consecutive rows of pts_sorted, which makes the gather coalesced;
 * the reference has no such variant (it always remaps first, pccnn_lib/pc/Neighborhood.py:47-53). */
int pccnn_compute_pdf_sorted(int manifold_dims, const float *bandwidth, const float *pts_sorted,
                             const float *samples, int64_t n, int d, const int32_t *neigh_sorted, int64_t t,
                             const int32_t *ends, float *pdf_out, void *stream);
/* The density of every point straight from the grid (d == 3): what Pointcloud.compute_pdf obtains from
 * find_neighbors (radius 4 x bandwidth, max_neighbors 300) followed by compute_pdf
 * (pccnn_lib/pc/Pointcloud.py:81-109), in one launch and without the pair list.  pts_sorted f32[n,3] and
 * sorted_keys i64[n] in key order; sample_order i32[n] (nullable) = original index of sorted point i, the row of
 * pdf_out it is written to; grid_ds / cell_table (nullable) / num_cells / radii (the search radii = cell size) as
 * for pccnn_find_neighbors_count.  With max_neighbors > 0 a point with more hits sums the subset that the capped
 * search keeps.  The terms and their order are those of pccnn_compute_pdf on that list.  pdf_norm_out (nullable)
 * f32[n] receives the estimate divided by the number of points of the point's cloud (pts_pdf_ of
 * Pointcloud.py:105-109). */
int pccnn_compute_pdf_grid(int manifold_dims, const float *bandwidth, const float *pts_sorted,
                           const int64_t *sorted_keys, int64_t n, const int32_t *sample_order,
                           const int32_t *grid_ds, int64_t num_pillars, const int32_t *cell_table,
                           int64_t total_cells, const int32_t *num_cells, const float *radii, int d,
                           int max_neighbors, float *pdf_out, float *pdf_norm_out, void *stream);
int pccnn_compute_pdf_grads(int manifold_dims, const float *bandwidth, const float *pts, int64_t n, int d,
                            const int32_t *neigh, int64_t t, const int32_t *ends, const float *in_grads,
                            float *pt_grads_out, void *stream);

/* ---- Poisson-disk selection --------------------------------------------
 * Replaces poisson_disk_sampling (pccnn_lib_ops/poisson_disk_sampling/poisson_disk_sampling.cuh:28-32,
 * poisson_disk_sampling.cu:110-196).  Inputs are in sorted-index space.
 * pccnn_poisson_disk_select writes selected_out i32[n] (0/1) and
 * selected_scan_out i32[n] (inclusive running count; last entry = S);
 * pccnn_compact_selected then writes the S selected indices, ascending, as i64. */
size_t pccnn_poisson_disk_workspace_bytes(int64_t n);
int pccnn_poisson_disk_select(const int64_t *sorted_keys, int64_t n, const int32_t *neigh, int64_t t,
                              const int32_t *ends, const int32_t *num_cells, int d,
                              int32_t *selected_out, int32_t *selected_scan_out,
                              void *workspace, size_t workspace_bytes, void *stream);
int pccnn_compact_selected(const int32_t *selected, const int32_t *selected_scan, int64_t n,
                           int64_t *ids_out, void *stream);
/* The same selection straight from the grid, without a neighbor list (d == 3): what PointPooling needs from
 * find_neighbors + poisson_disk_sampling (pccnn_lib/pc/PointPooling.py:58-65) in one call.  pts_sorted f32[n,3] and
 * sorted_keys in key order, grid_ds / cell_table (nullable) as for pccnn_find_neighbors_count, radii f32[3] = the
 * cell size.  Outputs and workspace as pccnn_poisson_disk_select; the result is identical to running that on the
 * uncapped self-neighborhood of the sorted points. */
int pccnn_poisson_disk_grid(const float *pts_sorted, const int64_t *sorted_keys, int64_t n,
                            const int32_t *grid_ds, int64_t num_pillars, const int32_t *cell_table,
                            int64_t total_cells, const int32_t *num_cells, const float *radii, int d,
                            int32_t *selected_out, int32_t *selected_scan_out,
                            void *workspace, size_t workspace_bytes, void *stream);

/* ---- host sequences with one read-back -----------------------------------
 * Chains of the entry points above for the steps whose output size depends on the data; each ends with one small
 * read-back and returns after it (the calls without "queued" in their name are synchronous).  The launches are those
 * of the entry points named.
 *
 * pccnn_bounding_box, and the box on the host as well (host_min_out / host_max_out: host memory, f32[batch_size,d]):
 * what pccnn_lib/pc/Grid.py:26-28 reads when it sizes a grid. */
int pccnn_bounding_box_host(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                            float *aabb_min_out, float *aabb_max_out, float *host_min_out, float *host_max_out,
                            void *stream);
/* pccnn_bounding_box with the host copy queued, not waited for: host_out is host memory of 2 * batch_size * d floats
 * and one int32, laid out as [minima | maxima | word].  With page-locked host_out and at most 256 box values the
 * kernels write host_out themselves (through its device address), the word - a 1 - last and behind a system-scope
 * fence, and *polled_out is 1: a caller that stored a negative value in the word before the call polls it.  Otherwise
 * *polled_out is 0, the boxes travel in two copies on `stream` and the caller waits for the stream (or an event). */
int pccnn_bounding_box_queued(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                              float *aabb_min_out, float *aabb_max_out, void *host_out, int *polled_out,
                              void *stream);
/* Poisson-disk pooling of a 3-D cloud up to the number of selected points: the grid of cell size `cell_size` over
 * the cloud (pccnn_grid_build, into the workspace), then pccnn_poisson_disk_grid, i.e. what
 * pccnn_lib/pc/PointPooling.py:38-65 does between the bounding box and the selected ids.  num_cells_host: the grid
 * size as three host ints (pccnn_num_cells' arithmetic on the host copy of the box); key_bits as pccnn_sort_keys;
 * with_cell_table != 0 builds the per-cell table for the walk.  Outputs: perm_out i32[n] (original index of sorted
 * point i), selected_out / selected_scan_out i32[n] as pccnn_poisson_disk_grid (sorted-index space), *count_out
 * (host) = number of selected points.  pooled_min_out / pooled_max_out (device, f32[batch_size,3]; all four NULL to
 * skip) receive the bounding box of the selected points per cloud, i.e. pccnn_bounding_box of the pooled cloud a
 * caller is about to build from them (pccnn_lib/pc/BoundingBox.py:17-18 on PointPooling's output), and
 * pooled_host_min_out / pooled_host_max_out (host) the same values, read back together with the count.
 * pccnn_compact_selected_remap then writes remap[i] of the selected i, ascending in i, as i64: with
 * remap = perm_out these are PointPooling's pooling_ids_ (PointPooling.py:66-69). */
size_t pccnn_pool_poisson_workspace_bytes(int64_t n, int64_t num_pillars, int64_t total_cells);
int pccnn_pool_poisson_select(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                              const float *aabb_min, const float *cell_size, const int32_t *num_cells_host,
                              int key_bits, int with_cell_table, int32_t *perm_out, int32_t *selected_out,
                              int32_t *selected_scan_out, int64_t *count_out, float *pooled_min_out,
                              float *pooled_max_out, float *pooled_host_min_out, float *pooled_host_max_out,
                              void *workspace, size_t workspace_bytes, void *stream);
/* pccnn_pool_poisson_select without the wait (n > 0, the boxes always): everything is queued on `stream`, ending
 * with the copy of the results to host_out - host memory of 6 * batch_size floats and one int32, best page-locked,
 * laid out as [minima f32[batch_size,3] | maxima f32[batch_size,3] | count i32] - and the call returns.  The caller
 * reads host_out once the work queued up to here has finished (an event recorded after the call, or a stream
 * synchronisation), and may queue other work on the stream in between; workspace and outputs stay untouched by
 * others until then.  The count is the last word to arrive (with page-locked host_out and up to 85 clouds the
 * kernels write host_out themselves, through its device address, the count behind a system-scope fence; otherwise
 * it travels in a copy of its own behind the boxes), so a caller that stored a negative value there before the call
 * may poll that word instead of waiting for an event.  *polled_out (host int, may be NULL) says which way the
 * results travel: 1 = written by the kernels, poll the count; 0 = copies, wait for the stream or an event.  No
 * counterpart in the reference, whose PointPooling waits where it reads the sizes. */
int pccnn_pool_poisson_select_queued(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                                     const float *aabb_min, const float *cell_size, const int32_t *num_cells_host,
                                     int key_bits, int with_cell_table, int32_t *perm_out, int32_t *selected_out,
                                     int32_t *selected_scan_out, float *pooled_min_out, float *pooled_max_out,
                                     void *host_out, int *polled_out, void *workspace, size_t workspace_bytes,
                                     void *stream);
int pccnn_compact_selected_remap(const int32_t *selected, const int32_t *selected_scan, const int32_t *remap,
                                 int64_t n, int64_t *ids_out, void *stream);
/* pccnn_compact_selected_remap with remap = perm, plus the rows a pooled cloud is made of: pooled_pts_out f32[S,d] =
 * pts[ids], pooled_batch_ids_out i32[S] = batch_ids[ids] (what PointPooling.pool_tensor returns for the cloud's own
 * coordinates and batch ids, pccnn_lib/pc/PointPooling.py:91-95). */
int pccnn_compact_pooled(const int32_t *selected, const int32_t *selected_scan, const int32_t *perm, const float *pts,
                         const int32_t *batch_ids, int64_t n, int d, int64_t *ids_out, float *pooled_pts_out,
                         int32_t *pooled_batch_ids_out, void *stream);
/* pccnn_grid_build for a grid whose size is known on the host (num_cells_host: d host ints): writes that size to
 * num_cells_out i32[d] on the device, where the kernels read it, instead of computing it there with pccnn_num_cells;
 * the numbers of pillars and cells follow from it.  with_cell_table != 0 (d == 3 only) fills cell_table_out
 * i32[cells + 1]. */
int pccnn_grid_build_sized(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                           const int32_t *num_cells_host, const float *cell_size, int64_t n, int d, int batch_size,
                           int key_bits, int with_cell_table, int32_t *num_cells_out, int64_t *keys_out,
                           int64_t *sorted_keys_out, int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out,
                           int32_t *cell_table_out, void *workspace, size_t workspace_bytes, void *stream);
/* The density of every point of a 3-D cloud from its box: pccnn_grid_build_sized (cell size = 4 x bandwidth, into
 * the workspace) and pccnn_compute_pdf_grid on it, i.e. the whole of pccnn_lib/pc/Pointcloud.py:81-109 after the
 * bounding box when no gradient is wanted.  No read-back: the call only queues work.  pdf_out / pdf_norm_out
 * (nullable) f32[n] in the cloud's own order. */
size_t pccnn_pdf_cloud_workspace_bytes(int64_t n, int64_t num_pillars, int64_t total_cells);
int pccnn_pdf_cloud(int manifold_dims, const float *bandwidth, const float *pts, const int32_t *batch_ids, int64_t n,
                    int batch_size, const float *aabb_min, const float *cell_size, const int32_t *num_cells_host,
                    int key_bits, int with_cell_table, int max_neighbors, float *pdf_out, float *pdf_norm_out,
                    void *workspace, size_t workspace_bytes, void *stream);
/* A layer's neighborhood up to the pair count (d == 3): pccnn_grid_build_sized over the cloud, keys and key order
 * of the samples (pccnn_compute_keys + pccnn_sort_keys into sample_keys_tmp i64[m] and sample_keys_out i64[m] /
 * sample_order_out i32[m] / sample_pts_out f32[m,3]; samples == NULL: the cloud itself, m == n, those four unused),
 * pccnn_find_neighbors_count, and the pair total in *total_out (host): what pccnn_lib/pc/layers/MCConv.py:136-140
 * and pccnn_lib/pc/Neighborhood.py:27-45 do up to the allocation of the pair list.  sort_workspace as
 * pccnn_grid_build for max(n, m) keys, workspace as pccnn_find_neighbors_count; pccnn_find_neighbors_fill then takes
 * the same sorted points, sample buffers, tables and workspace. */
int pccnn_neighborhood_count(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                             const float *aabb_min, const float *cell_size, const int32_t *num_cells_host,
                             int key_bits, int with_cell_table, int32_t *num_cells_out, int64_t *keys_out,
                             int64_t *sorted_keys_out, int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out,
                             int32_t *cell_table_out, const float *samples, const int32_t *sample_batch_ids, int64_t m,
                             int64_t *sample_keys_tmp, int64_t *sample_keys_out, int32_t *sample_order_out,
                             float *sample_pts_out, int max_neighbors, int32_t *ends_out, int64_t *total_out,
                             void *sort_workspace, size_t sort_workspace_bytes, void *workspace, size_t workspace_bytes,
                             void *stream);

/* ---- convolutions -------------------------------------------------------
 * Shapes: pts f32[n,d], feats f32[n,c_in], samples f32[m,d], neigh i32[t,2]
 * (point, sample), ends i32[m], radii f32[d] (device), out f32[m,c_out].
 *
 * KPConv replaces kp_conv / kp_conv_grads (pccnn_lib_ops/pcconvs/kpconv.cuh:32-67,
 * kpconv.cu:32-112): kernel_pts f32[k,d], weights f32[k*c_in, c_out] with row
 * f*k + kk.  Backward outputs: d_weights f32[k*c_in,c_out], d_feats f32[n,c_in],
 * d_kernel_pts f32[k,d], d_pts f32[n,d], d_samples f32[m,d].
 *
 * MCConv replaces mc_conv / mc_conv_grads (pccnn_lib_ops/pcconvs/mcconv.cuh:32-69,
 * mcconv.cu:32-143): pdf f32[n], axis f32[d,k], bias f32[k] with k = hidden*num_mlps,
 * weights f32[num_mlps, k*c_in/num_mlps, c_out/num_mlps].  Backward outputs:
 * d_weights (same shape), d_feats, d_axis f32[d,k], d_bias f32[k], d_pdf f32[n],
 * d_pts, d_samples.
 *
 * 1 <= k <= 64.  2 <= d <= 6 (the reference's tests run the convolutions in 2, 3 and 4 dimensions,
 * unit_test/utest_kpconv.ini, utest_mcconv.ini).  d == 3 runs kernels that fuse the basis into the gather; any other
 * d evaluates the basis per pair into f32[t,k] in the workspace, runs the convolution on it as a caller-given basis
 * and maps the basis gradient back per pair.  For d != 3 the forward calls need a workspace too
 * (pccnn_conv_workspace_bytes(..., backward = 0)) and `mirror` is ignored.
 *
 * Three arguments go beyond the reference's interface.  `proj_out` / `proj` (nullable): the projection
 * P f32[m, c_in, k] (k fastest) that the forward call builds on its way to `out`; a caller that keeps it
 * (proj_out != NULL) can hand it to the backward call, which otherwise rebuilds it like the reference does
 * (kpconv.cu:78-87).  `grad_mask`: which gradients to produce (PCCNN_GRAD_* bits; PCCNN_GRAD_ALL is the
 * reference's behaviour).  Requested outputs are fully overwritten; outputs not requested may be NULL and are
 * not touched.  `mirror` (nullable, i32[t]): for a symmetric neighborhood (the samples are the points, so
 * n == m, and the search was not capped) the index of pair (b, a) for every pair (a, b), from
 * pccnn_mirror_pairs; with it d_pts and d_pdf are summed per point in a fixed order instead of with float
 * atomics (the reference scatters with index_add_ atomics, pt_diff.cu:51-80). */
#define PCCNN_GRAD_WEIGHTS 1
#define PCCNN_GRAD_FEATS 2
#define PCCNN_GRAD_BASIS_PARAMS 4 /* d_kernel_pts, or d_axis and d_bias */
#define PCCNN_GRAD_PDF 8
#define PCCNN_GRAD_PTS 16         /* d_pts and d_samples */
#define PCCNN_GRAD_ALL 31
/* A flag beside the groups (not part of PCCNN_GRAD_ALL): run the backward pass without float atomics, so that every
 * result is bit-identical from run to run.  The reference accumulates with atomics (gpuAtomicAdd,
 * pccnn_lib_ops/pcconvs/shared/feat_basis_proj_grads.cu:132,146; index_add_, pt_diff.cu:51-80); so does this library
 * by default, because it is faster.  With the flag, the feature gradient of every pair is stored as a row of its own
 * and the rows of a point are summed in a fixed order: through `mirror` when it is given, else through a by-point
 * index of the pair list that the call builds in its workspace (a key sort of the t pairs); d_pts / d_pdf take the
 * same route, and the basis-parameter partial sums are kept per sample.  3-D (or caller-given basis) only; the
 * workspace must hold pccnn_conv_workspace_bytes_deterministic(...) bytes. */
#define PCCNN_GRAD_DETERMINISTIC 32
size_t pccnn_conv_workspace_bytes(int64_t m, int64_t t, int c_in, int k, int c_out, int backward);
size_t pccnn_conv_workspace_bytes_deterministic(int64_t n, int64_t m, int64_t t, int c_in, int k, int c_out);
/* mirror_out i32[t]: index of the pair (point b, sample a) for pair t = (point a, sample b), -1 when absent;
 * *missing_out i32 = number of pairs without a mirror (0 for a symmetric neighborhood). */
int pccnn_mirror_pairs(const int32_t *neigh, const int32_t *ends, int64_t t, int64_t m, int32_t *mirror_out,
                       int32_t *missing_out, void *stream);
int pccnn_kpconv_forward(const float *pts, const float *feats, const float *samples, const int32_t *neigh,
                         const int32_t *ends, const float *radii, const float *kernel_pts, float sigma,
                         const float *weights, int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int c_out,
                         float *out, float *proj_out, void *workspace, size_t workspace_bytes, void *stream);
int pccnn_kpconv_backward(const float *pts, const float *feats, const float *samples, const int32_t *neigh,
                          const int32_t *ends, const float *radii, const float *kernel_pts, float sigma,
                          const float *weights, const float *in_grads, const float *proj, const int32_t *mirror,
                          int grad_mask, int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int c_out,
                          float *d_weights, float *d_feats, float *d_kernel_pts, float *d_pts, float *d_samples,
                          void *workspace, size_t workspace_bytes, void *stream);
int pccnn_mcconv_forward(const float *pts, const float *pdf, const float *feats, const float *samples,
                         const int32_t *neigh, const int32_t *ends, const float *radii, const float *axis,
                         const float *bias, const float *weights,
                         int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int num_mlps, int c_out,
                         float *out, float *proj_out, void *workspace, size_t workspace_bytes, void *stream);
int pccnn_mcconv_backward(const float *pts, const float *pdf, const float *feats, const float *samples,
                          const int32_t *neigh, const int32_t *ends, const float *radii, const float *axis,
                          const float *bias, const float *weights, const float *in_grads, const float *proj,
                          const int32_t *mirror, int grad_mask,
                          int64_t n, int64_t m, int64_t t, int d, int c_in, int k, int num_mlps, int c_out,
                          float *d_weights, float *d_feats, float *d_axis, float *d_bias, float *d_pdf,
                          float *d_pts, float *d_samples,
                          void *workspace, size_t workspace_bytes, void *stream);

/* An optional forward path that keeps the projection on chip: with pccnn_set_fused_forward(1), forward calls that are
 * not asked for the projection (proj_out == NULL) and whose shape allows it (3-D or caller-given basis, k <= 16,
 * num_mlps == 1, c_in > 32, c_out 64, 128 or 256) run as one kernel that gathers a 64-sample x 256-column slice of P
 * into LDS and multiplies it with the matching rows of the weights right away, where the reference writes P out and
 * reads it back for torch::matmul (pccnn_lib_ops/pcconvs/kpconv.cu:52-57, mcconv.cu:58-68).  Same results to rounding.
 * Off by default: on MI355X the two-kernel path is faster (csrc/conv_fused.hip has the figures).  Returns the
 * previous setting.  Process-wide. */
int pccnn_set_fused_forward(int on);

/* ---- the other convolution families -----------------------------------------
 * One descriptor-driven triple covers KPConvN, PCCNN, PointConv and SPHConv (and, redundantly, KPConv and
 * MCConv).  It replaces kp_conv_n* (pccnn_lib_ops/pcconvs/kpconvn.cuh:32-93), pccnn* (pccnn.cuh:32-93),
 * point_conv / point_conv_grads / point_conv_weight_var (pointconv.cuh:37-56) and sph_conv*
 * (sphconv.cuh:19-55); they differ only in the basis evaluated per pair and in SPHConv's division of the
 * output by the neighbor count (`divide_by_count`).
 *
 *   kind       a                      b               c             other fields
 *   KP         kernel_pts f32[k,d]    -               -             sigma
 *   MLP        axis f32[d,k]          bias f32[k]     -             pdf f32[n]
 *   KPN        kernel_pts f32[k,d]    -               -             sigma, pdf      (KP value / pdf)
 *   GAUSS      kernel_pts f32[k,d]    -               -             sigma, pdf      (exp(-|kp-d|^2/(2 sigma^2)) / pdf)
 *   EXPLICIT   basis f32[t,k]         -               -             (values given per pair: PointConv)
 *   SPH        radial edges f32[nb0]  azimuth [nb1]   polar [nb2]   k is nb0*nb1*nb2 + 1 (one-hot spherical bin; d == 3 only)
 *
 * Backward outputs: d_param_a = d_kernel_pts [k,d] (KP, KPN, GAUSS), d_axis [d,k] (MLP) or the basis gradient
 * f32[t,k] (EXPLICIT); d_param_b = d_bias [k] (MLP); d_pdf only for MLP and GAUSS; d_pts / d_samples for the
 * kinds whose basis depends on the positions (not EXPLICIT, not SPH).  Groups a kind does not have are ignored. */
#define PCCNN_BASIS_KP 0
#define PCCNN_BASIS_MLP 1
#define PCCNN_BASIS_KPN 2
#define PCCNN_BASIS_GAUSS 3
#define PCCNN_BASIS_EXPLICIT 4
#define PCCNN_BASIS_SPH 5
typedef struct pccnn_basis {
    int kind;
    int k;
    const float *a, *b, *c;
    int nb0, nb1, nb2;
    float sigma;
    const float *pdf;
} pccnn_basis;
int pccnn_conv_forward(const pccnn_basis *basis, const float *pts, const float *feats, const float *samples,
                       const int32_t *neigh, const int32_t *ends, const float *radii, const float *weights,
                       int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps, int c_out, int divide_by_count,
                       float *out, float *proj_out, void *workspace, size_t workspace_bytes, void *stream);
int pccnn_conv_backward(const pccnn_basis *basis, const float *pts, const float *feats, const float *samples,
                        const int32_t *neigh, const int32_t *ends, const float *radii, const float *weights,
                        const float *in_grads, const float *proj, const int32_t *mirror, int grad_mask,
                        int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps, int c_out, int divide_by_count,
                        float *d_weights, float *d_feats, float *d_param_a, float *d_param_b, float *d_pdf,
                        float *d_pts, float *d_samples, void *workspace, size_t workspace_bytes, void *stream);
int pccnn_conv_weight_var(const pccnn_basis *basis, const float *pts, const float *feats, const float *samples,
                          const int32_t *neigh, const int32_t *ends, const float *radii,
                          int64_t n, int64_t m, int64_t t, int d, int c_in, int divide_by_count, float *out,
                          void *workspace, size_t workspace_bytes, void *stream);

/* PointConv's per-pair basis op and its gradient: replaces point_conv_basis / point_conv_basis_grads
 * (pccnn_lib_ops/pcconvs/pointconv.cuh:20-35): basis_out f32[t,k] = ((pts[n_t] - samples[s_t]) / radii) . axis + bias;
 * backward: d_pts f32[n,d], d_samples f32[m,d], d_axis f32[d,k], d_bias f32[k] from basis_grads f32[t,k]. */
int pccnn_linear_basis_forward(const float *pts, const float *samples, const int32_t *neigh, const float *radii,
                               const float *axis, const float *bias, int64_t n, int64_t m, int64_t t, int d, int k,
                               float *basis_out, void *stream);
size_t pccnn_linear_basis_workspace_bytes(int64_t t);
int pccnn_linear_basis_backward(const float *pts, const float *samples, const int32_t *neigh, const float *radii,
                                const float *axis, const float *bias, const float *basis_grads,
                                int64_t n, int64_t m, int64_t t, int d, int k,
                                float *d_pts, float *d_samples, float *d_axis, float *d_bias,
                                void *workspace, size_t workspace_bytes, void *stream);

/* ---- variance statistic of the weight initialisation -----------------------
 * Replaces kp_conv_weight_var / mc_conv_weight_var (pccnn_lib_ops/pcconvs/kpconv.cuh:82-90, mcconv.cuh:83-92;
 * kernel pccnn_lib_ops/pcconvs/shared/compute_variance_weights.cu:24-170): out[0] (one float, device) =
 * 1 / mean over the samples of sum_{i,j in N(s)} (w_i . w_j)(F_i . F_j), evaluated as the squared norm of the
 * sample's projection tile.  Same tensor arguments as the forward calls, without the weights. */
size_t pccnn_conv_weight_var_workspace_bytes(int64_t m, int64_t t, int c_in, int k);
int pccnn_kpconv_weight_var(const float *pts, const float *feats, const float *samples, const int32_t *neigh,
                            const int32_t *ends, const float *radii, const float *kernel_pts, float sigma,
                            int64_t n, int64_t m, int64_t t, int d, int c_in, int k, float *out,
                            void *workspace, size_t workspace_bytes, void *stream);
int pccnn_mcconv_weight_var(const float *pts, const float *pdf, const float *feats, const float *samples,
                            const int32_t *neigh, const int32_t *ends, const float *radii, const float *axis,
                            const float *bias, int64_t n, int64_t m, int64_t t, int d, int c_in, int k, float *out,
                            void *workspace, size_t workspace_bytes, void *stream);

/* ---- dense contraction --------------------------------------------------
 * The fp32 MFMA GEMM the convolutions use for the [M, K*Cin] x [K*Cin, Cout]
 * contraction (torch::matmul at pccnn_lib_ops/pcconvs/kpconv.cu:56-57,90-96 and
 * mcconv.cu:64-68,111-120), exposed for tests and benchmarks.
 * C[batch][rows,cols] = op(A) * op(B) with inner size `inner`; row-major storage,
 * a_trans: A stored [inner, rows]; b_trans: B stored [cols, inner]; lda/ldb/ldc are
 * row strides in elements, stride_* batch strides in elements.  split_k > 1
 * needs workspace of batch*split_k*rows*cols floats. */
int pccnn_gemm_f32(const float *a, const float *b, float *c, int64_t rows, int64_t cols, int64_t inner,
                   int a_trans, int b_trans, int64_t lda, int64_t ldb, int64_t ldc,
                   int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                   int split_k, void *workspace, size_t workspace_bytes, void *stream);

/* ---- bf16 contraction ----------------------------------------------------
 * A mode the reference does not have (its contraction is an fp32 torch::matmul, mcconv.cu:64-68,111-120,
 * kpconv.cu:56-57,90-96): the operands of the three contractions of a convolution -- the projection P, the
 * weights and the output gradients -- are rounded to bf16 (nearest even) and multiplied on the bf16 matrix
 * pipe with fp32 accumulation; bases, aggregation, every result and every other gradient stay fp32.
 * pccnn_conv_forward_bf16 / pccnn_conv_backward_bf16 take the arguments of pccnn_conv_forward /
 * pccnn_conv_backward, except that the projection handed from forward to backward is uint16_t[m, c_in*k] of
 * bf16 bit patterns; workspace size as for the fp32 calls.
 * pccnn_gemm_bf16 is that contraction on its own (arguments as pccnn_gemm_f32, A and B bf16 bit patterns, C fp32);
 * pccnn_f32_to_bf16 is the rounding the library applies (dst[i] = bf16(src[i])). */
int pccnn_f32_to_bf16(const float *src, uint16_t *dst, int64_t count, void *stream);
int pccnn_gemm_bf16(const uint16_t *a, const uint16_t *b, float *c, int64_t rows, int64_t cols, int64_t inner,
                    int a_trans, int b_trans, int64_t lda, int64_t ldb, int64_t ldc,
                    int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                    int split_k, void *workspace, size_t workspace_bytes, void *stream);
int pccnn_conv_forward_bf16(const pccnn_basis *basis, const float *pts, const float *feats, const float *samples,
                            const int32_t *neigh, const int32_t *ends, const float *radii, const float *weights,
                            int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps, int c_out,
                            int divide_by_count, float *out, uint16_t *proj_out,
                            void *workspace, size_t workspace_bytes, void *stream);
int pccnn_conv_backward_bf16(const pccnn_basis *basis, const float *pts, const float *feats, const float *samples,
                             const int32_t *neigh, const int32_t *ends, const float *radii, const float *weights,
                             const float *in_grads, const uint16_t *proj, const int32_t *mirror, int grad_mask,
                             int64_t n, int64_t m, int64_t t, int d, int c_in, int num_mlps, int c_out,
                             int divide_by_count, float *d_weights, float *d_feats, float *d_param_a,
                             float *d_param_b, float *d_pdf, float *d_pts, float *d_samples,
                             void *workspace, size_t workspace_bytes, void *stream);

/* ---- per-kernel timing ---------------------------------------------------
 * Measurement hooks with no counterpart in the reference (it has no profiler hooks).  While
 * enabled, the entry points above bracket their main kernels with HIP events on the launch
 * stream; pccnn_timing_read waits for the recorded events and returns, for timer `id` in
 * [0, pccnn_timing_count()), the number of bracketed launches and their summed duration in ms
 * since the last reset.  Timer names: pccnn_timing_name(id).  Off by default. */
int pccnn_timing_enable(int on);
int pccnn_timing_reset(void);
int pccnn_timing_count(void);
const char *pccnn_timing_name(int id);
int pccnn_timing_read(int id, int64_t *h_launches, double *h_total_ms);

/* Measurement helper with no counterpart in the reference: copies `count` floats (a multiple of 4, 16-byte
 * aligned pointers) with plain loads and stores.  A profiler's memory-traffic counters read for this kernel,
 * whose traffic is known (4*count bytes each way), give the scale for the same counters on the other kernels. */
int pccnn_calibration_copy(const float *src, float *dst, int64_t count, void *stream);

/* Row permutation, used where the reference's Python gathers with torch.index_select (e.g. pccnn_lib/pc/Grid.py:68-70
 * for the sorted copies): dst f32[rows, row_floats] = src[index[i], :], index i32[rows] with values in
 * [0, src_rows) (a row whose index is outside is left untouched).  And the inverse of a permutation of 0..n-1:
 * inverse[perm[i]] = i. */
int pccnn_gather_rows_f32(const float *src, const int32_t *index, float *dst, int64_t rows, int row_floats,
                          int64_t src_rows, void *stream);
int pccnn_invert_permutation_i32(const int32_t *perm, int32_t *inverse, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PCCNN_HIP_H */
