// Poisson-disk selection over points in sorted (cell-key) order.
// 2^D launches, one per cell-parity colour.  Cells of one colour are at least two cells apart in every direction,
// so they never share a neighbor and can be processed concurrently; inside a cell the points are taken in sorted
// order, and a point is selected iff none of its listed neighbors is selected yet.
//
// One wavefront per cell, one point per lane (64 at a time).  Every lane scans its own neighbor list: a neighbor
// outside the current 64 points is settled already (an earlier colour, an earlier round of this cell) or still
// unselected, so its flag in memory decides; a neighbor among the current 64 with a smaller index is noted in a
// 64-bit mask.  The serial part of the greedy rule is then a scalar loop over the candidates in order: candidate i
// is selected iff none of its noted neighbors was selected before it.  The result is that of the one-thread-per-
// cell walk of the reference (poisson_disk_sampling.cu:56-105), with the latency of a cell's ~10^3 dependent
// loads paid across 64 lanes.
#include "common.h"
#include "grid_walk.h"

// Also clears what the passes start from: the selection flags and (when given) the 64 counters.
__global__ void __launch_bounds__(256)
cell_flag_kernel(const int64_t *__restrict__ keys, int64_t n, int32_t *__restrict__ flags,
                 int32_t *__restrict__ selected, int32_t *__restrict__ counters)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (counters != nullptr && i < 64) counters[i] = 0;
    if (i < n) {
        flags[i] = (i == 0 || keys[i - 1] != keys[i]) ? 1 : 0;
        selected[i] = 0;
    }
}

// cell_first[c] = index of the first point of the c-th non-empty cell; *count = number of such cells.
__global__ void __launch_bounds__(256)
cell_list_kernel(const int32_t *__restrict__ flags, const int32_t *__restrict__ scan, int64_t n,
                 int32_t *__restrict__ cell_first, int32_t *__restrict__ count)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    if (flags[i] != 0) cell_first[scan[i] - 1] = (int32_t)i;
    if (i == n - 1) *count = scan[i];
}

// Three dimensions: the non-empty cells listed per parity colour, so that a pass only touches the cells it works
// on.  colour_list[colour * n + i] = (index into cell_first, first point, key) of the i-th cell of that colour - what
// a pass needs to start on a cell, in one 16-byte load instead of three dependent ones -, in no particular
// order: cells of one colour do not interact, so the selection does not depend on the order.  colour_count[8]
// must be zero on entry.  The kernel writes the list of first points and the number of cells as well (what
// cell_list_kernel does for the other dimensions).
// COLOUR_ITEMS points per thread: 8 on large inputs, where the atomics on the eight global counters would
// otherwise queue up, 1 on small ones, where the launch is a single round of short workgroups.
template <int COLOUR_ITEMS>
__global__ void __launch_bounds__(256)
cell_colour_kernel(const int32_t *__restrict__ flags, const int32_t *__restrict__ scan, const int64_t *__restrict__ keys,
                   int64_t n, const int32_t *__restrict__ num_cells, int4 *__restrict__ colour_list,
                   int32_t *__restrict__ colour_count, int32_t *__restrict__ cell_first, int32_t *__restrict__ count)
{
    // the workgroup counts its cells per colour in LDS and reserves its share of every list with one atomic
    __shared__ int local[8], start[8];
    if (threadIdx.x < 8) local[threadIdx.x] = 0;
    __syncthreads();
    const int nc0 = num_cells[0], nc1 = num_cells[1], nc2 = num_cells[2];
    int colour[COLOUR_ITEMS], at[COLOUR_ITEMS];
#pragma unroll
    for (int r = 0; r < COLOUR_ITEMS; ++r) {
        const int64_t i = ((int64_t)blockIdx.x * COLOUR_ITEMS + r) * 256 + threadIdx.x;
        colour[r] = -1;
        at[r] = 0;
        if (i == n - 1) *count = scan[i];
        if (i < n && flags[i] != 0) {
            cell_first[scan[i] - 1] = (int32_t)i;
            long long k = keys[i];
            const int c2 = (int)(k % nc2); k /= nc2;
            const int c1 = (int)(k % nc1); k /= nc1;
            const int c0 = (int)(k % nc0);
            colour[r] = (c0 & 1) | ((c1 & 1) << 1) | ((c2 & 1) << 2);
            at[r] = atomicAdd(&local[colour[r]], 1);
        }
    }
    __syncthreads();
    if (threadIdx.x < 8) start[threadIdx.x] = local[threadIdx.x] ? atomicAdd(&colour_count[threadIdx.x], local[threadIdx.x]) : 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < COLOUR_ITEMS; ++r) {
        const int64_t i = ((int64_t)blockIdx.x * COLOUR_ITEMS + r) * 256 + threadIdx.x;
        if (colour[r] >= 0) {
            const long long k = keys[i];
            colour_list[(int64_t)colour[r] * n + start[colour[r]] + at[r]] =
                make_int4(scan[i] - 1, (int)i, (int)(k & 0xffffffffll), (int)(k >> 32));
        }
    }
}

#define POISSON_LOADS 8     // neighbor flags requested together by a lane

template <int D>
__global__ void __launch_bounds__(256)
poisson_pass_kernel(const int64_t *__restrict__ keys, int64_t n, const int2 *__restrict__ neigh,
                    const int32_t *__restrict__ ends, const int32_t *__restrict__ num_cells, int colour,
                    volatile int32_t *used, const int32_t *__restrict__ cell_first,
                    const int32_t *__restrict__ cell_count)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const int cells = *cell_count;
    const int32_t *settled = (const int32_t *)used;
    int nc[D];
#pragma unroll
    for (int k = 0; k < D; ++k) nc[k] = num_cells[k];
    for (int64_t c = wave; c < cells; c += waves) {
        const int first = cell_first[c];
        const int last = (c + 1 < cells) ? cell_first[c + 1] : (int)n;      // one past the cell's last point
        long long aux = keys[first];
        bool mine = true;
#pragma unroll
        for (int k = D - 1; k >= 0; --k) {
            const int cc = (int)(aux % nc[k]);
            aux /= nc[k];
            mine = mine && ((cc % 2) == ((colour >> k) & 1));
        }
        if (!mine) continue;                                                // uniform: one key per wavefront
        for (int base = first; base < last; base += 64) {
            const int p = base + lane;
            const bool valid = p < last;
            bool cand = valid;
            unsigned long long earlier = 0ull;      // neighbors among the current 64 points that come before p
            if (valid) {
                const int lo = p > 0 ? ends[p - 1] : 0;
                const int hi = ends[p];
                for (int t = lo; t < hi && cand; t += POISSON_LOADS) {
                    int q[POISSON_LOADS], u[POISSON_LOADS];
#pragma unroll
                    for (int v = 0; v < POISSON_LOADS; ++v) q[v] = (t + v < hi) ? neigh[t + v].x : p;
#pragma unroll
                    for (int v = 0; v < POISSON_LOADS; ++v) {
                        const bool in_round = q[v] >= base && q[v] < p;
                        // Flags of other cells were written by earlier launches (cells of one colour are never
                        // neighbors), so an ordinary cached load sees them; only an earlier round of this very
                        // cell, written by this wavefront a moment ago, has to be read past the caches.
                        if (in_round || q[v] == p) u[v] = 0;
                        else if (q[v] >= first && q[v] < base) u[v] = used[q[v]];
                        else u[v] = settled[q[v]];
                        if (in_round) earlier |= 1ull << (q[v] - base);
                    }
#pragma unroll
                    for (int v = 0; v < POISSON_LOADS; ++v) cand = cand && (u[v] == 0);
                }
            }
            // the greedy rule among the current points, in order
            unsigned long long todo = __ballot(cand);
            unsigned long long selected = 0ull;
            while (todo != 0ull) {
                const int i = __ffsll((long long)todo) - 1;
                todo &= todo - 1ull;
                const unsigned lo32 = (unsigned)__builtin_amdgcn_readlane((int)(earlier & 0xffffffffull), i);
                const unsigned hi32 = (unsigned)__builtin_amdgcn_readlane((int)(earlier >> 32), i);
                const unsigned long long before = ((unsigned long long)hi32 << 32) | lo32;
                if ((before & selected) == 0ull) selected |= 1ull << i;
            }
            if (valid && ((selected >> lane) & 1ull)) used[p] = 1;
            // a later round of this cell reads these flags back
            if (base + 64 < last) __threadfence();
        }
    }
}

// The same selection without a neighbor list (three dimensions).  A point can only be blocked by a point that is
// already selected, and those are few: so instead of testing every candidate of the 27-cell walk against every point,
// the wavefront of a cell reads the selection flags of the walk's index ranges (contiguous, 64 per load), and only
// for the flagged candidates fetches the position and tests it against the cell's points, one per lane.  Neighbors
// inside the cell are found by testing the cell's points against each other, and the greedy rule is resolved on the
// masks as above.  The predicate is the neighbor search's, un-contracted fp32, with the deciding point in the role of
// the sample (it is symmetric: the differences only change sign).
struct PoissonGridArgs {
    const float *pts;            // sorted points [n,3]
    GridRef grid;
    const int32_t *num_cells;    // [3]
    const float *radii;          // [3]
    volatile int32_t *used;      // [n] selection flags
    const int32_t *cell_first;   // compact list of the non-empty cells
    const int32_t *cell_count;
    const int4 *colour_list;     // [8][n] cells per parity colour: (index into cell_first, first point, key lo, key hi)
    const int32_t *colour_count; // [8]
};

__global__ void __launch_bounds__(256)
poisson_grid_pass_kernel(PoissonGridArgs a, int colour)
{
#pragma clang fp contract(off)
    __shared__ int2 rng[4][9];
    const int lane = threadIdx.x & 63;
    const int wib = threadIdx.x >> 6;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const int cells = *a.cell_count;
    const int mine = a.colour_count[colour];                   // cells of this pass's colour
    const int32_t *settled = (const int32_t *)a.used;
    const int nc0 = a.num_cells[0], nc1 = a.num_cells[1], nc2 = a.num_cells[2];
    const float ir0 = __fdiv_rn(1.0f, a.radii[0]);
    const float ir1 = __fdiv_rn(1.0f, a.radii[1]);
    const float ir2 = __fdiv_rn(1.0f, a.radii[2]);
    for (int64_t ci = wave; ci < mine; ci += waves) {
        const int4 rec = a.colour_list[(int64_t)colour * a.grid.n + ci];
        const int c = rec.x, first = rec.y;
        const int last = (c + 1 < cells) ? a.cell_first[c + 1] : (int)a.grid.n;
        long long k = ((long long)rec.w << 32) | (unsigned int)rec.z;
        const int c2 = (int)(k % nc2); k /= nc2;
        const int c1 = (int)(k % nc1);
        const long long pil = k; k /= nc1;
        const int c0 = (int)(k % nc0);
        // the nine index ranges of the 27-cell walk (lane o looks up range o)
        if (lane < 9) {
            const int cmin = c2 > 0 ? c2 - 1 : 0, cmax = c2 + 1 < nc2 ? c2 + 1 : nc2 - 1;
            const int dx = lane / 3 - 1, dy = lane % 3 - 1;
            const int x = c0 + dx, y = c1 + dy;
            int f = 0, l = 0;
            if (x >= 0 && x < nc0 && y >= 0 && y < nc1)
                grid_pillar_range(a.grid, pil + (long long)dx * nc1 + dy, nc2, cmin, cmax, f, l);
            rng[wib][lane] = make_int2(f, l);
        }
        for (int base = first; base < last; base += 64) {
            const int p = base + lane;
            const bool valid = p < last;
            float sx = 0.f, sy = 0.f, sz = 0.f;
            if (valid) { sx = a.pts[(int64_t)p * 3 + 0]; sy = a.pts[(int64_t)p * 3 + 1]; sz = a.pts[(int64_t)p * 3 + 2]; }
            bool cand = valid;
            // Selected points around the cell: flags first, positions only where a flag is set.  The first 64 flags of
            // all nine ranges are requested together, then every lane that found a flag fetches that point's position
            // itself, so the tests below read registers: two memory round trips per round of 64 points, not one or
            // two per range.
            int flag[9];
            float fx[9], fy[9], fz[9];
#pragma unroll
            for (int r = 0; r < 9; ++r) {
                const int2 g = rng[wib][r];
                const int q = g.x + lane;
                flag[r] = 0;
                if (lane < g.y) flag[r] = (q >= first && q < base) ? a.used[q] : settled[q];
            }
#pragma unroll
            for (int r = 0; r < 9; ++r) {
                fx[r] = fy[r] = fz[r] = 0.f;
                if (flag[r] != 0) {
                    const int64_t q = (int64_t)rng[wib][r].x + lane;
                    fx[r] = a.pts[q * 3 + 0]; fy[r] = a.pts[q * 3 + 1]; fz[r] = a.pts[q * 3 + 2];
                }
            }
#pragma unroll
            for (int r = 0; r < 9; ++r) {
                unsigned long long set = __ballot(flag[r] != 0);
                while (set != 0ull) {
                    const int src = __builtin_ctzll(set);
                    set &= set - 1ull;
                    const float vx = (sx - pccnn_bcast_f(fx[r], src)) * ir0;
                    const float vy = (sy - pccnn_bcast_f(fy[r], src)) * ir1;
                    const float vz = (sz - pccnn_bcast_f(fz[r], src)) * ir2;
                    const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                    if (acc < 1.0f) cand = false;
                }
            }
            // ranges of more than 64 points: the rest, range by range
            for (int r = 0; r < 9; ++r) {
                const int2 g = rng[wib][r];
                for (int j0 = 64; j0 < g.y; j0 += 64) {
                    const int q = g.x + j0 + lane;
                    int more = 0;
                    if (j0 + lane < g.y) more = (q >= first && q < base) ? a.used[q] : settled[q];
                    unsigned long long set = __ballot(more != 0);
                    while (set != 0ull) {
                        const int qi = g.x + j0 + __builtin_ctzll(set);
                        set &= set - 1ull;
                        const float vx = (sx - a.pts[(int64_t)qi * 3 + 0]) * ir0;
                        const float vy = (sy - a.pts[(int64_t)qi * 3 + 1]) * ir1;
                        const float vz = (sz - a.pts[(int64_t)qi * 3 + 2]) * ir2;
                        const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                        if (acc < 1.0f) cand = false;
                    }
                }
            }
            // neighbors among the current points that come before p
            unsigned long long earlier = 0ull;
            const int cnt = (last - base) < 64 ? (last - base) : 64;
            for (int i = 0; i + 1 < cnt; ++i) {
                const float qx = pccnn_bcast_f(sx, i), qy = pccnn_bcast_f(sy, i), qz = pccnn_bcast_f(sz, i);
                const float vx = (sx - qx) * ir0;
                const float vy = (sy - qy) * ir1;
                const float vz = (sz - qz) * ir2;
                const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                if (i < lane && acc < 1.0f) earlier |= 1ull << i;
            }
            // the greedy rule among the current points, in order
            unsigned long long todo = __ballot(cand);
            unsigned long long selected = 0ull;
            while (todo != 0ull) {
                const int i = __ffsll((long long)todo) - 1;
                todo &= todo - 1ull;
                const unsigned lo32 = (unsigned)__builtin_amdgcn_readlane((int)(earlier & 0xffffffffull), i);
                const unsigned hi32 = (unsigned)__builtin_amdgcn_readlane((int)(earlier >> 32), i);
                const unsigned long long before = ((unsigned long long)hi32 << 32) | lo32;
                if ((before & selected) == 0ull) selected |= 1ull << i;
            }
            if (valid && ((selected >> lane) & 1ull)) a.used[p] = 1;
            if (base + 64 < last) __threadfence();
        }
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
    if (n < 1) n = 1;
    // scan scratch | cell flags | first point of every cell | cell count, colour counts | 16-byte cell records per colour (3-D)
    return pccnn_align(pccnn_scan_tmp_elems(n) * sizeof(int32_t)) + 2 * pccnn_align((size_t)n * sizeof(int32_t)) + 512 +
           pccnn_align(8 * (size_t)n * 4 * sizeof(int32_t));
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
    PccnnArena arena(workspace, workspace_bytes);
    int32_t *scan_tmp = arena.take<int32_t>(pccnn_scan_tmp_elems(n));
    int32_t *flags = arena.take<int32_t>((size_t)n);
    int32_t *cell_first = arena.take<int32_t>((size_t)n);
    int32_t *cell_count = arena.take<int32_t>(1);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_poisson_disk_select: workspace of %zu bytes, need %zu",
                  workspace_bytes, pccnn_poisson_disk_workspace_bytes(n));
    // the list of non-empty cells (selected_scan_out is free until the end and holds the scan of the flags)
    const unsigned blocks = (unsigned)pccnn_ceil_div(n, 256);
    cell_flag_kernel<<<blocks, 256, 0, s>>>(sorted_keys, n, flags, selected_out, nullptr);
    PCCNN_LAUNCH_CHECK();
    int rc = pccnn_scan_inclusive_i32(flags, selected_scan_out, n, 0, scan_tmp, s);
    if (rc != PCCNN_OK) return rc;
    cell_list_kernel<<<blocks, 256, 0, s>>>(flags, selected_scan_out, n, cell_first, cell_count);
    PCCNN_LAUNCH_CHECK();
    // a fixed number of wavefronts takes the cells in turn: the cell count stays on the device
    int64_t pass_blocks = pccnn_ceil_div(n, 64);
    if (pass_blocks > 2048) pass_blocks = 2048;
    for (int colour = 0; colour < (1 << d); ++colour) {
        PCCNN_DIM_DISPATCH(d, poisson_pass_kernel, <<<(unsigned)pass_blocks, 256, 0, s>>>(
            sorted_keys, n, (const int2 *)neigh, ends, num_cells, colour, selected_out, cell_first, cell_count));
        PCCNN_LAUNCH_CHECK();
    }
    return pccnn_scan_inclusive_i32(selected_out, selected_scan_out, n, 0, scan_tmp, s);
}

extern "C" int pccnn_poisson_disk_grid(const float *pts_sorted, const int64_t *sorted_keys, int64_t n,
                                       const int32_t *grid_ds, int64_t num_pillars, const int32_t *cell_table,
                                       int64_t total_cells, const int32_t *num_cells, const float *radii, int d,
                                       int32_t *selected_out, int32_t *selected_scan_out, void *workspace,
                                       size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(d == 3, PCCNN_ERR_UNSUPPORTED, "pccnn_poisson_disk_grid: d=%d is not supported (3 only)", d);
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31) && num_pillars >= 0, PCCNN_ERR_INVALID,
                  "pccnn_poisson_disk_grid: n=%lld num_pillars=%lld", (long long)n, (long long)num_pillars);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(pts_sorted && sorted_keys && grid_ds && num_cells && radii && selected_out && selected_scan_out,
                  PCCNN_ERR_INVALID, "pccnn_poisson_disk_grid: null pointer");
    PCCNN_REQUIRE(cell_table == nullptr || total_cells > 0, PCCNN_ERR_INVALID,
                  "pccnn_poisson_disk_grid: a cell table needs its size");
    hipStream_t s = (hipStream_t)stream;
    PccnnArena arena(workspace, workspace_bytes);
    int32_t *scan_tmp = arena.take<int32_t>(pccnn_scan_tmp_elems(n));
    int32_t *flags = arena.take<int32_t>((size_t)n);
    int32_t *cell_first = arena.take<int32_t>((size_t)n);
    int32_t *cell_count = arena.take<int32_t>(64);               // [0]: cells; [8..15]: cells per colour
    int4 *colour_list = arena.take<int4>(8 * (size_t)n);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_poisson_disk_grid: workspace of %zu bytes, need %zu",
                  workspace_bytes, pccnn_poisson_disk_workspace_bytes(n));
    int32_t *colour_count = cell_count + 8;
    const unsigned blocks = (unsigned)pccnn_ceil_div(n, 256);
    cell_flag_kernel<<<blocks, 256, 0, s>>>(sorted_keys, n, flags, selected_out, cell_count);
    PCCNN_LAUNCH_CHECK();
    int rc = pccnn_scan_inclusive_i32(flags, selected_scan_out, n, 0, scan_tmp, s);
    if (rc != PCCNN_OK) return rc;
    if (n > 131072)
        cell_colour_kernel<8><<<(unsigned)pccnn_ceil_div(n, 256 * 8), 256, 0, s>>>(
            flags, selected_scan_out, sorted_keys, n, num_cells, colour_list, colour_count, cell_first, cell_count);
    else
        cell_colour_kernel<1><<<blocks, 256, 0, s>>>(flags, selected_scan_out, sorted_keys, n, num_cells, colour_list,
                                                     colour_count, cell_first, cell_count);
    PCCNN_LAUNCH_CHECK();
    PoissonGridArgs a;
    a.pts = pts_sorted;
    a.grid = GridRef{cell_table, total_cells, grid_ds, num_pillars, sorted_keys, n};
    a.num_cells = num_cells; a.radii = radii; a.used = selected_out;
    a.cell_first = cell_first; a.cell_count = cell_count;
    a.colour_list = colour_list; a.colour_count = colour_count;
    int64_t pass_blocks = pccnn_ceil_div(n, 64);
    if (pass_blocks > 2048) pass_blocks = 2048;
    for (int colour = 0; colour < 8; ++colour) {
        poisson_grid_pass_kernel<<<(unsigned)pass_blocks, 256, 0, s>>>(a, colour);
        PCCNN_LAUNCH_CHECK();
    }
    return pccnn_scan_inclusive_i32(selected_out, selected_scan_out, n, 0, scan_tmp, s);
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
