// Host-side sequences for the steps of a hierarchy level whose sizes depend on data: the box of a cloud, the
// Poisson-disk pooling of a cloud, and the pair count of a neighborhood.  Each is a fixed chain of the library's
// own launches with one small read-back at its end; run from Python, such a chain of 10 - 30 launches over a cloud
// of a few thousand points costs several times more in interpreter and binding overhead than on the GPU.  Nothing
// here computes: the kernels are those of the entry points that are called.
//
// The read-backs go through a small pinned host buffer (one per host thread, allocated on first use and kept):
// an asynchronous copy into it on the caller's stream, then a wait for that stream - or, where the last kernel of
// the chain can write the result itself (the pair total, the pooled boxes and their count, a cloud's box), a store
// into page-locked host memory through its device address and a host that polls the word written last.
#include "common.h"
#include <string.h>
#include <chrono>

namespace {

struct PinnedSlot {
    void *p = nullptr;
    size_t bytes = 0;
};
thread_local PinnedSlot g_slot;

int pinned_slot(size_t bytes, void **out)
{
    if (g_slot.bytes < bytes) {
        if (g_slot.p) PCCNN_HIP_CHECK(hipHostFree(g_slot.p));
        g_slot.p = nullptr;
        g_slot.bytes = 0;
        const size_t want = bytes < 4096 ? 4096 : bytes;
        PCCNN_HIP_CHECK(hipHostMalloc(&g_slot.p, want, hipHostMallocPortable));
        g_slot.bytes = want;
    }
    *out = g_slot.p;
    return PCCNN_OK;
}

// device -> caller's host memory, through the pinned buffer; returns when the values are there
int read_back(void *host_out, const void *dev, size_t bytes, hipStream_t s)
{
    void *slot;
    int rc = pinned_slot(bytes, &slot);
    if (rc != PCCNN_OK) return rc;
    PCCNN_HIP_CHECK(hipMemcpyAsync(slot, dev, bytes, hipMemcpyDeviceToHost, s));
    PCCNN_HIP_CHECK(hipStreamSynchronize(s));
    memcpy(host_out, slot, bytes);
    return PCCNN_OK;
}

// checks a grid size given on the host and derives the numbers of pillars and cells
int grid_extent(const char *who, const int32_t *num_cells_host, int d, int batch_size, int64_t *num_pillars,
                int64_t *total_cells)
{
    int64_t total = batch_size;
    for (int k = 0; k < d; ++k) {
        const int c = num_cells_host[k];
        PCCNN_REQUIRE(c > 0, PCCNN_ERR_INVALID, "%s: %d cells along axis %d", who, c, k);
        PCCNN_REQUIRE(total <= INT64_MAX / c, PCCNN_ERR_INVALID, "%s: the cell count overflows 64 bits", who);
        total *= c;
    }
    *num_pillars = (int64_t)batch_size * num_cells_host[0] * num_cells_host[1];
    *total_cells = total;
    return PCCNN_OK;
}

__global__ void __launch_bounds__(256)
compact_remap_kernel(const int32_t *__restrict__ flags, const int32_t *__restrict__ scan,
                     const int32_t *__restrict__ remap, int64_t n, int64_t *__restrict__ ids)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && flags[i] != 0) ids[scan[i] - 1] = remap[i];
}

// the selected points' original indices, coordinates and batch ids, in the order of the selection
__global__ void __launch_bounds__(256)
compact_pooled_kernel(const int32_t *__restrict__ flags, const int32_t *__restrict__ scan,
                      const int32_t *__restrict__ perm, const float *__restrict__ pts,
                      const int32_t *__restrict__ batch_ids, int64_t n, int d, int64_t *__restrict__ ids,
                      float *__restrict__ pts_out, int32_t *__restrict__ batch_out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n || flags[i] == 0) return;
    const int64_t j = scan[i] - 1, o = perm[i];
    ids[j] = o;
    for (int k = 0; k < d; ++k) pts_out[j * d + k] = pts[o * d + k];
    batch_out[j] = batch_ids[o];
}

struct PoolLayout {
    int64_t *keys, *sorted_keys;
    float *sorted_pts;
    int32_t *grid_ds, *cell_table, *num_cells;
    void *sort_ws, *poisson_ws;
    size_t sort_bytes, poisson_bytes;
};

bool pool_layout(PccnnArena &arena, int64_t n, int64_t num_pillars, int64_t total_cells, PoolLayout &l)
{
    l.keys = arena.take<int64_t>((size_t)n);
    l.sorted_keys = arena.take<int64_t>((size_t)n);
    l.sorted_pts = arena.take<float>((size_t)n * 3);
    l.grid_ds = arena.take<int32_t>((size_t)num_pillars * 2);
    l.cell_table = total_cells > 0 ? arena.take<int32_t>((size_t)total_cells + 1) : nullptr;
    l.num_cells = arena.take<int32_t>(64);
    l.sort_bytes = pccnn_grid_build_workspace_bytes(n);
    l.sort_ws = arena.take<char>(l.sort_bytes);
    l.poisson_bytes = pccnn_poisson_disk_workspace_bytes(n);
    l.poisson_ws = arena.take<char>(l.poisson_bytes);
    return arena.ok();
}

}  // namespace

extern "C" int pccnn_bounding_box_host(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                                       float *aabb_min_out, float *aabb_max_out, float *host_min_out,
                                       float *host_max_out, void *stream)
{
    PCCNN_REQUIRE(host_min_out && host_max_out, PCCNN_ERR_INVALID, "pccnn_bounding_box_host: null host pointer");
    int rc = pccnn_bounding_box(pts, batch_ids, n, d, batch_size, aabb_min_out, aabb_max_out, stream);
    if (rc != PCCNN_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    const size_t bytes = (size_t)batch_size * d * sizeof(float);
    void *slot;
    if ((rc = pinned_slot(2 * bytes, &slot)) != PCCNN_OK) return rc;
    PCCNN_HIP_CHECK(hipMemcpyAsync(slot, aabb_min_out, bytes, hipMemcpyDeviceToHost, s));
    PCCNN_HIP_CHECK(hipMemcpyAsync((char *)slot + bytes, aabb_max_out, bytes, hipMemcpyDeviceToHost, s));
    PCCNN_HIP_CHECK(hipStreamSynchronize(s));
    memcpy(host_min_out, slot, bytes);
    memcpy(host_max_out, (char *)slot + bytes, bytes);
    return PCCNN_OK;
}

extern "C" int pccnn_bounding_box_queued(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                                         float *aabb_min_out, float *aabb_max_out, void *host_out, int *polled_out,
                                         void *stream)
{
    PCCNN_REQUIRE(host_out && polled_out, PCCNN_ERR_INVALID, "pccnn_bounding_box_queued: null host pointer");
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS && batch_size > 0, PCCNN_ERR_INVALID,
                  "pccnn_bounding_box_queued: d=%d batch_size=%d", d, batch_size);
    *polled_out = 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t bytes = (size_t)batch_size * d * sizeof(float);
    // page-locked host memory and one workgroup's worth of box values: the kernel that pads the boxes writes them
    // to host_out itself and a 1 behind them, last; otherwise two copies, and the caller waits for the stream
    void *host_on_device = nullptr;
    bool direct = batch_size * d <= 256;
    if (direct && hipHostGetDevicePointer(&host_on_device, host_out, 0) != hipSuccess) {
        (void)hipGetLastError();
        direct = false;
    }
    PccnnBoxMask mask;
    if (direct) mask.tail = (float *)host_on_device;
    int rc = pccnn_bounding_box_masked(pts, batch_ids, n, d, batch_size, aabb_min_out, aabb_max_out, mask, stream);
    if (rc != PCCNN_OK) return rc;
    if (!direct) {
        PCCNN_HIP_CHECK(hipMemcpyAsync(host_out, aabb_min_out, bytes, hipMemcpyDeviceToHost, s));
        PCCNN_HIP_CHECK(hipMemcpyAsync((char *)host_out + bytes, aabb_max_out, bytes, hipMemcpyDeviceToHost, s));
    }
    *polled_out = direct ? 1 : 0;
    return PCCNN_OK;
}

extern "C" size_t pccnn_pool_poisson_workspace_bytes(int64_t n, int64_t num_pillars, int64_t total_cells)
{
    if (n < 1) n = 1;
    if (num_pillars < 1) num_pillars = 1;
    return 2 * pccnn_align((size_t)n * sizeof(int64_t)) + pccnn_align((size_t)n * 3 * sizeof(float)) +
           pccnn_align((size_t)num_pillars * 2 * sizeof(int32_t)) +
           (total_cells > 0 ? pccnn_align(((size_t)total_cells + 1) * sizeof(int32_t)) : 0) + 256 +
           pccnn_align(pccnn_grid_build_workspace_bytes(n)) + pccnn_align(pccnn_poisson_disk_workspace_bytes(n));
}

// Grid, Poisson-disk selection, the selection's size and (with_box) the selected points' boxes, all queued on the
// stream and ending with the copies that bring the results to `host_dst`: [minima | maxima | count (int32)] with
// the boxes, the count alone without.  Nothing waits here.
static int pool_select_queue(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                             const float *aabb_min, const float *cell_size, const int32_t *num_cells_host,
                             int key_bits, int with_cell_table, int32_t *perm_out, int32_t *selected_out,
                             int32_t *selected_scan_out, float *pooled_min_out, float *pooled_max_out, bool with_box,
                             void *host_dst, int *polled_out, void *workspace, size_t workspace_bytes, hipStream_t s)
{
    const char *who = "pccnn_pool_poisson_select";
    if (polled_out) *polled_out = 0;
    PCCNN_REQUIRE(pts && batch_ids && aabb_min && cell_size && perm_out && selected_out && selected_scan_out,
                  PCCNN_ERR_INVALID, "%s: null pointer", who);
    for (int k = 0; k < 3; ++k)
        PCCNN_REQUIRE(num_cells_host[k] > 0, PCCNN_ERR_INVALID, "%s: %d cells along axis %d", who, num_cells_host[k], k);
    int64_t num_pillars = (int64_t)batch_size * num_cells_host[0] * num_cells_host[1];
    int64_t total_cells = with_cell_table ? num_pillars * num_cells_host[2] : 0;
    PccnnArena arena(workspace, workspace_bytes);
    PoolLayout l;
    PCCNN_REQUIRE(pool_layout(arena, n, num_pillars, total_cells, l), PCCNN_ERR_WORKSPACE,
                  "%s: workspace of %zu bytes, need %zu", who, workspace_bytes,
                  pccnn_pool_poisson_workspace_bytes(n, num_pillars, total_cells));
    void *stream = (void *)s;
    int rc = pccnn_grid_build_sized(pts, batch_ids, aabb_min, num_cells_host, cell_size, n, 3, batch_size, key_bits,
                                    with_cell_table, l.num_cells, l.keys, l.sorted_keys, perm_out, l.sorted_pts,
                                    l.grid_ds, l.cell_table, l.sort_ws, l.sort_bytes, stream);
    if (rc != PCCNN_OK) return rc;
    rc = pccnn_poisson_disk_grid(l.sorted_pts, l.sorted_keys, n, l.grid_ds, num_pillars, l.cell_table, total_cells,
                                 l.num_cells, cell_size, 3, selected_out, selected_scan_out, l.poisson_ws,
                                 l.poisson_bytes, stream);
    if (rc != PCCNN_OK) return rc;
    if (!with_box) {
        PCCNN_HIP_CHECK(hipMemcpyAsync(host_dst, selected_scan_out + (n - 1), sizeof(int32_t), hipMemcpyDeviceToHost, s));
        return PCCNN_OK;
    }
    // The box of the selected points, from the sorted copy and the selection flags.  The kernel that pads the boxes
    // also writes them, and behind them the count, to a second place.  With page-locked `host_dst` that place is
    // host_dst itself, through its address on the device: nothing is copied, and because the count is written last,
    // behind a system-scope fence, the caller may poll that word.  Otherwise (or with more than 256 box values, which
    // the padding kernel writes from several workgroups) the second place is a stretch of the workspace (the
    // unsorted keys are not needed any more) that one copy brings over, and the count follows in a copy of its own,
    // so that it still arrives last.
    const size_t box = (size_t)batch_size * 3 * sizeof(float);
    void *host_on_device = nullptr;
    bool direct = batch_size * 3 <= 256;
    if (direct && hipHostGetDevicePointer(&host_on_device, host_dst, 0) != hipSuccess) {
        (void)hipGetLastError();                        // pageable memory: not an error, the copies do it
        direct = false;
    }
    const bool staged = !direct && 2 * box + sizeof(int32_t) <= pccnn_align((size_t)n * sizeof(int64_t));
    PccnnBoxMask mask;
    mask.selected = selected_out;
    mask.perm = perm_out;
    if (direct) {
        mask.tail = (float *)host_on_device;
        mask.count_src = selected_scan_out + (n - 1);
    } else if (staged) {
        mask.tail = (float *)l.keys;
    }
    rc = pccnn_bounding_box_masked(l.sorted_pts, batch_ids, n, 3, batch_size, pooled_min_out, pooled_max_out, mask,
                                   stream);
    if (rc != PCCNN_OK) {
        // a launch that writes into the caller's host block may already be queued: let it land before the caller
        // hears of the error and reuses the block
        if (direct) (void)hipStreamSynchronize(s);
        return rc;
    }
    if (direct) {
        if (polled_out) *polled_out = 1;
        return PCCNN_OK;
    }
    if (staged) {
        PCCNN_HIP_CHECK(hipMemcpyAsync(host_dst, mask.tail, 2 * box, hipMemcpyDeviceToHost, s));
    } else {
        PCCNN_HIP_CHECK(hipMemcpyAsync(host_dst, pooled_min_out, box, hipMemcpyDeviceToHost, s));
        PCCNN_HIP_CHECK(hipMemcpyAsync((char *)host_dst + box, pooled_max_out, box, hipMemcpyDeviceToHost, s));
    }
    PCCNN_HIP_CHECK(hipMemcpyAsync((char *)host_dst + 2 * box, selected_scan_out + (n - 1), sizeof(int32_t),
                                   hipMemcpyDeviceToHost, s));
    return PCCNN_OK;
}

extern "C" int pccnn_pool_poisson_select(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                                         const float *aabb_min, const float *cell_size,
                                         const int32_t *num_cells_host, int key_bits, int with_cell_table,
                                         int32_t *perm_out, int32_t *selected_out, int32_t *selected_scan_out,
                                         int64_t *count_out, float *pooled_min_out, float *pooled_max_out,
                                         float *pooled_host_min_out, float *pooled_host_max_out, void *workspace,
                                         size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31) && batch_size > 0, PCCNN_ERR_INVALID,
                  "pccnn_pool_poisson_select: n=%lld batch_size=%d", (long long)n, batch_size);
    PCCNN_REQUIRE(count_out && num_cells_host, PCCNN_ERR_INVALID, "pccnn_pool_poisson_select: null host pointer");
    const bool with_box = pooled_min_out != nullptr;
    PCCNN_REQUIRE(!with_box || (pooled_max_out && pooled_host_min_out && pooled_host_max_out), PCCNN_ERR_INVALID,
                  "pccnn_pool_poisson_select: the box of the selection needs all four of its outputs");
    *count_out = 0;
    if (n == 0) return PCCNN_OK;
    hipStream_t s = (hipStream_t)stream;
    const size_t box = with_box ? (size_t)batch_size * 3 * sizeof(float) : 0;
    void *slot;
    int rc;
    if ((rc = pinned_slot(2 * box + sizeof(int32_t), &slot)) != PCCNN_OK) return rc;
    rc = pool_select_queue(pts, batch_ids, n, batch_size, aabb_min, cell_size, num_cells_host, key_bits,
                           with_cell_table, perm_out, selected_out, selected_scan_out, pooled_min_out, pooled_max_out,
                           with_box, slot, nullptr, workspace, workspace_bytes, s);
    if (rc != PCCNN_OK) return rc;
    PCCNN_HIP_CHECK(hipStreamSynchronize(s));           // count and box: one wait
    int32_t count;
    if (with_box) {
        memcpy(pooled_host_min_out, slot, box);
        memcpy(pooled_host_max_out, (char *)slot + box, box);
    }
    memcpy(&count, (char *)slot + 2 * box, sizeof(int32_t));
    *count_out = count;
    return PCCNN_OK;
}

extern "C" int pccnn_pool_poisson_select_queued(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                                                const float *aabb_min, const float *cell_size,
                                                const int32_t *num_cells_host, int key_bits, int with_cell_table,
                                                int32_t *perm_out, int32_t *selected_out, int32_t *selected_scan_out,
                                                float *pooled_min_out, float *pooled_max_out, void *host_out,
                                                int *polled_out, void *workspace, size_t workspace_bytes,
                                                void *stream)
{
    PCCNN_REQUIRE(n > 0 && n < (1ll << 31) && batch_size > 0, PCCNN_ERR_INVALID,
                  "pccnn_pool_poisson_select_queued: n=%lld batch_size=%d", (long long)n, batch_size);
    PCCNN_REQUIRE(host_out && num_cells_host && pooled_min_out && pooled_max_out, PCCNN_ERR_INVALID,
                  "pccnn_pool_poisson_select_queued: null pointer");
    return pool_select_queue(pts, batch_ids, n, batch_size, aabb_min, cell_size, num_cells_host, key_bits,
                             with_cell_table, perm_out, selected_out, selected_scan_out, pooled_min_out, pooled_max_out,
                             true, host_out, polled_out, workspace, workspace_bytes, (hipStream_t)stream);
}

extern "C" int pccnn_compact_selected_remap(const int32_t *selected, const int32_t *selected_scan,
                                            const int32_t *remap, int64_t n, int64_t *ids_out, void *stream)
{
    PCCNN_REQUIRE(n >= 0, PCCNN_ERR_INVALID, "pccnn_compact_selected_remap: n=%lld", (long long)n);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(selected && selected_scan && remap && ids_out, PCCNN_ERR_INVALID,
                  "pccnn_compact_selected_remap: null pointer");
    compact_remap_kernel<<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(selected, selected_scan,
                                                                                           remap, n, ids_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" int pccnn_compact_pooled(const int32_t *selected, const int32_t *selected_scan, const int32_t *perm,
                                    const float *pts, const int32_t *batch_ids, int64_t n, int d, int64_t *ids_out,
                                    float *pooled_pts_out, int32_t *pooled_batch_ids_out, void *stream)
{
    PCCNN_REQUIRE(n >= 0 && d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_INVALID, "pccnn_compact_pooled: n=%lld d=%d",
                  (long long)n, d);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(selected && selected_scan && perm && pts && batch_ids && ids_out && pooled_pts_out &&
                      pooled_batch_ids_out,
                  PCCNN_ERR_INVALID, "pccnn_compact_pooled: null pointer");
    compact_pooled_kernel<<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(
        selected, selected_scan, perm, pts, batch_ids, n, d, ids_out, pooled_pts_out, pooled_batch_ids_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" size_t pccnn_pdf_cloud_workspace_bytes(int64_t n, int64_t num_pillars, int64_t total_cells)
{
    if (n < 1) n = 1;
    if (num_pillars < 1) num_pillars = 1;
    // keys, sorted keys | sorted points | permutation | pillar table | cell table | grid size | sort scratch
    return 2 * pccnn_align((size_t)n * sizeof(int64_t)) + pccnn_align((size_t)n * 3 * sizeof(float)) +
           pccnn_align((size_t)n * sizeof(int32_t)) + pccnn_align((size_t)num_pillars * 2 * sizeof(int32_t)) +
           (total_cells > 0 ? pccnn_align(((size_t)total_cells + 1) * sizeof(int32_t)) : 0) + 256 +
           pccnn_align(pccnn_grid_build_workspace_bytes(n));
}

extern "C" int pccnn_pdf_cloud(int manifold_dims, const float *bandwidth, const float *pts, const int32_t *batch_ids,
                               int64_t n, int batch_size, const float *aabb_min, const float *cell_size,
                               const int32_t *num_cells_host, int key_bits, int with_cell_table, int max_neighbors,
                               float *pdf_out, float *pdf_norm_out, void *workspace, size_t workspace_bytes,
                               void *stream)
{
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31) && batch_size > 0 && num_cells_host, PCCNN_ERR_INVALID,
                  "pccnn_pdf_cloud: n=%lld batch_size=%d", (long long)n, batch_size);
    if (n == 0) return PCCNN_OK;
    for (int k = 0; k < 3; ++k)
        PCCNN_REQUIRE(num_cells_host[k] > 0, PCCNN_ERR_INVALID, "pccnn_pdf_cloud: %d cells along axis %d",
                      num_cells_host[k], k);
    const int64_t num_pillars = (int64_t)batch_size * num_cells_host[0] * num_cells_host[1];
    const int64_t total_cells = with_cell_table ? num_pillars * num_cells_host[2] : 0;
    PccnnArena arena(workspace, workspace_bytes);
    int64_t *keys = arena.take<int64_t>((size_t)n);
    int64_t *sorted_keys = arena.take<int64_t>((size_t)n);
    float *sorted_pts = arena.take<float>((size_t)n * 3);
    int32_t *perm = arena.take<int32_t>((size_t)n);
    int32_t *grid_ds = arena.take<int32_t>((size_t)num_pillars * 2);
    int32_t *cell_table = total_cells > 0 ? arena.take<int32_t>((size_t)total_cells + 1) : nullptr;
    int32_t *num_cells = arena.take<int32_t>(64);
    const size_t sort_bytes = pccnn_grid_build_workspace_bytes(n);
    void *sort_ws = arena.take<char>(sort_bytes);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_pdf_cloud: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_pdf_cloud_workspace_bytes(n, num_pillars, total_cells));
    int rc = pccnn_grid_build_sized(pts, batch_ids, aabb_min, num_cells_host, cell_size, n, 3, batch_size, key_bits,
                                    with_cell_table, num_cells, keys, sorted_keys, perm, sorted_pts, grid_ds, cell_table,
                                    sort_ws, sort_bytes, stream);
    if (rc != PCCNN_OK) return rc;
    return pccnn_compute_pdf_grid(manifold_dims, bandwidth, sorted_pts, sorted_keys, n, perm, grid_ds, num_pillars,
                                  cell_table, total_cells, num_cells, cell_size, 3, max_neighbors, pdf_out, pdf_norm_out,
                                  stream);
}

extern "C" int pccnn_grid_build_sized(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                                      const int32_t *num_cells_host, const float *cell_size, int64_t n, int d,
                                      int batch_size, int key_bits, int with_cell_table, int32_t *num_cells_out,
                                      int64_t *keys_out, int64_t *sorted_keys_out, int32_t *perm_out,
                                      float *sorted_pts_out, int32_t *grid_ds_out, int32_t *cell_table_out,
                                      void *workspace, size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_grid_build_sized: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(num_cells_host && num_cells_out && batch_size > 0, PCCNN_ERR_INVALID,
                  "pccnn_grid_build_sized: null grid size or batch_size=%d", batch_size);
    PCCNN_REQUIRE(!with_cell_table || (cell_table_out && d == 3), PCCNN_ERR_INVALID,
                  "pccnn_grid_build_sized: the cell table needs its output and d == 3");
    int64_t num_pillars, total_cells;
    int rc = grid_extent("pccnn_grid_build_sized", num_cells_host, d, batch_size, &num_pillars, &total_cells);
    if (rc != PCCNN_OK) return rc;
    if (d == 3 && n > 0)
        return pccnn_grid_build_sized3(pts, batch_ids, aabb_min, num_cells_host, cell_size, n, key_bits, num_pillars,
                                       with_cell_table ? total_cells : 0, num_cells_out, keys_out, sorted_keys_out,
                                       perm_out, sorted_pts_out, grid_ds_out, with_cell_table ? cell_table_out : nullptr,
                                       workspace, workspace_bytes, stream);
    rc = pccnn_compute_keys_sized(pts, batch_ids, aabb_min, num_cells_host, cell_size, n, d, num_cells_out, keys_out,
                                  (hipStream_t)stream);
    if (rc != PCCNN_OK) return rc;
    return pccnn_grid_build_from_keys(keys_out, pts, num_cells_out, n, d, key_bits, num_pillars,
                                      with_cell_table ? total_cells : 0, sorted_keys_out, perm_out, sorted_pts_out,
                                      grid_ds_out, with_cell_table ? cell_table_out : nullptr, workspace,
                                      workspace_bytes, stream);
}

extern "C" int pccnn_neighborhood_count(const float *pts, const int32_t *batch_ids, int64_t n, int batch_size,
                                        const float *aabb_min, const float *cell_size,
                                        const int32_t *num_cells_host, int key_bits, int with_cell_table,
                                        int32_t *num_cells_out, int64_t *keys_out, int64_t *sorted_keys_out,
                                        int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out,
                                        int32_t *cell_table_out, const float *samples,
                                        const int32_t *sample_batch_ids, int64_t m, int64_t *sample_keys_tmp,
                                        int64_t *sample_keys_out, int32_t *sample_order_out, float *sample_pts_out,
                                        int max_neighbors, int32_t *ends_out, int64_t *total_out,
                                        void *sort_workspace, size_t sort_workspace_bytes, void *workspace,
                                        size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(total_out, PCCNN_ERR_INVALID, "pccnn_neighborhood_count: null host pointer");
    *total_out = 0;
    PCCNN_REQUIRE(n > 0 && m > 0, PCCNN_ERR_INVALID, "pccnn_neighborhood_count: n=%lld m=%lld (both must be positive)",
                  (long long)n, (long long)m);
    int rc = pccnn_grid_build_sized(pts, batch_ids, aabb_min, num_cells_host, cell_size, n, 3, batch_size, key_bits,
                                    with_cell_table, num_cells_out, keys_out, sorted_keys_out, perm_out, sorted_pts_out,
                                    grid_ds_out, cell_table_out, sort_workspace, sort_workspace_bytes, stream);
    if (rc != PCCNN_OK) return rc;
    const int64_t num_pillars = (int64_t)batch_size * num_cells_host[0] * num_cells_host[1];
    const int64_t total_cells = with_cell_table ? num_pillars * num_cells_host[2] : 0;
    const float *s_pts = sorted_pts_out;
    const int64_t *s_keys = sorted_keys_out;
    const int32_t *s_order = perm_out;
    if (samples != nullptr) {
        PCCNN_REQUIRE(sample_batch_ids && sample_keys_tmp && sample_keys_out && sample_order_out && sample_pts_out,
                      PCCNN_ERR_INVALID, "pccnn_neighborhood_count: null sample buffer");
        // (the keys of the samples are computed by their sort's first histogram pass)
        PccnnKeySource src = {samples, sample_batch_ids, aabb_min, cell_size, num_cells_out, {}, nullptr, 0};
        rc = pccnn_sort_keys_from_points(src, sample_keys_tmp, m, key_bits, sample_keys_out, sample_order_out,
                                         sample_pts_out, sort_workspace, sort_workspace_bytes, stream);
        if (rc != PCCNN_OK) return rc;
        s_pts = sample_pts_out;
        s_keys = sample_keys_out;
        s_order = sample_order_out;
    } else {
        PCCNN_REQUIRE(m == n, PCCNN_ERR_INVALID, "pccnn_neighborhood_count: without samples m must equal n");
    }
    // The scan that ends the count writes the 64-bit pair total straight into the pinned host buffer (mapped into
    // the device's address space), and the host polls that word: no copy launch behind the scan and no wake-up
    // through the runtime.  Should the word not arrive (it always has), the stream is waited for as before.
    void *slot, *slot_on_device;
    if ((rc = pinned_slot(sizeof(int64_t), &slot)) != PCCNN_OK) return rc;
    PCCNN_HIP_CHECK(hipHostGetDevicePointer(&slot_on_device, slot, 0));
    volatile int64_t *word = (volatile int64_t *)slot;
    const int64_t pending = INT64_MIN;
    *word = pending;
    pccnn_redirect_pair_total((int64_t *)slot_on_device);
    rc = pccnn_find_neighbors_count(sorted_pts_out, sorted_keys_out, n, s_pts, s_keys, m, s_order, 1, grid_ds_out,
                                    num_pillars, with_cell_table ? cell_table_out : nullptr, total_cells, num_cells_out,
                                    cell_size, 3, max_neighbors, ends_out, workspace, workspace_bytes, stream);
    pccnn_redirect_pair_total(nullptr);
    if (rc != PCCNN_OK) {
        // a launch that writes the total into this thread's pinned word may already be queued: let it land before
        // the next call arms the word again
        (void)hipStreamSynchronize((hipStream_t)stream);
        return rc;
    }
    const auto start = std::chrono::steady_clock::now();
    unsigned spins = 0;
    while (*word == pending) {
        if ((++spins & 1023u) == 0 && std::chrono::steady_clock::now() - start > std::chrono::milliseconds(20)) {
            PCCNN_HIP_CHECK(hipStreamSynchronize((hipStream_t)stream));
            break;
        }
    }
    const int64_t total = *word;
    PCCNN_REQUIRE(total != pending, PCCNN_ERR_INVALID, "pccnn_neighborhood_count: the pair total did not arrive");
    *total_out = total;
    return PCCNN_OK;
}
