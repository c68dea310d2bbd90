// Poisson-disk selection over points in sorted (cell-key) order.
// 2^D launches, one per cell-parity colour.  Cells of one colour are at least two cells apart
// in every direction, so they never share a neighbor and can be processed concurrently; inside
// a cell the points are visited serially in sorted order by the thread that owns the cell's
// first point, and a point is selected iff none of its listed neighbors is selected yet.
#include "common.h"

template <int D>
__global__ void __launch_bounds__(256)
poisson_pass_kernel(const int64_t *__restrict__ keys, int64_t n, const int2 *__restrict__ neigh,
                    const int32_t *__restrict__ ends, const int32_t *__restrict__ num_cells, int colour,
                    volatile int32_t *used)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long long key = keys[i];
    if (i > 0 && keys[i - 1] == key) return;          // not the first point of its cell
    long long aux = key;
    bool mine = true;
#pragma unroll
    for (int k = D - 1; k >= 0; --k) {
        const int nc = num_cells[k];
        const int c = (int)(aux % nc);
        aux /= nc;
        mine = mine && ((c % 2) == ((colour >> k) & 1));
    }
    if (!mine) return;
    for (int64_t p = i; p < n && keys[p] == key; ++p) {
        const int lo = p > 0 ? ends[p - 1] : 0;
        const int hi = ends[p];
        bool free_spot = true;
        for (int t = lo; t < hi && free_spot; ++t) free_spot = used[neigh[t].x] == 0;
        if (free_spot) used[p] = 1;
    }
}

__global__ void __launch_bounds__(256)
compact_kernel(const int32_t *__restrict__ flags, const int32_t *__restrict__ scan, int64_t n,
               int64_t *__restrict__ ids)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && flags[i] != 0) ids[scan[i] - 1] = i;
}

extern "C" size_t pccnn_poisson_disk_workspace_bytes(int64_t n)
{
    return pccnn_align(pccnn_scan_tmp_elems(n) * sizeof(int32_t)) + 256;
}

extern "C" int pccnn_poisson_disk_select(const int64_t *sorted_keys, int64_t n, const int32_t *neigh, int64_t t,
                                         const int32_t *ends, const int32_t *num_cells, int d,
                                         int32_t *selected_out, int32_t *selected_scan_out, void *workspace,
                                         size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_poisson_disk_select: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(n >= 0 && t >= 0 && n < (1ll << 31), PCCNN_ERR_INVALID, "pccnn_poisson_disk_select: n=%lld t=%lld",
                  (long long)n, (long long)t);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(sorted_keys && ends && num_cells && selected_out && selected_scan_out && (t == 0 || neigh),
                  PCCNN_ERR_INVALID, "pccnn_poisson_disk_select: null pointer");
    PCCNN_REQUIRE(workspace && workspace_bytes >= pccnn_poisson_disk_workspace_bytes(n), PCCNN_ERR_WORKSPACE,
                  "pccnn_poisson_disk_select: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_poisson_disk_workspace_bytes(n));
    hipStream_t s = (hipStream_t)stream;
    int rc = pccnn_fill_i32(selected_out, 0, n, s);
    if (rc != PCCNN_OK) return rc;
    for (int colour = 0; colour < (1 << d); ++colour) {
        PCCNN_DIM_DISPATCH(d, poisson_pass_kernel, <<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, s>>>(
            sorted_keys, n, (const int2 *)neigh, ends, num_cells, colour, selected_out));
        PCCNN_LAUNCH_CHECK();
    }
    return pccnn_scan_inclusive_i32(selected_out, selected_scan_out, n, 0, (int32_t *)workspace, s);
}

extern "C" int pccnn_compact_selected(const int32_t *selected, const int32_t *selected_scan, int64_t n,
                                      int64_t *ids_out, void *stream)
{
    PCCNN_REQUIRE(n >= 0, PCCNN_ERR_INVALID, "pccnn_compact_selected: n=%lld", (long long)n);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(selected && selected_scan && ids_out, PCCNN_ERR_INVALID, "pccnn_compact_selected: null pointer");
    compact_kernel<<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(selected, selected_scan, n,
                                                                                     ids_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}
