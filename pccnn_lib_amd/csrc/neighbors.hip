// Radius neighbor search on the pillar grid: count pass, device scan, fill pass.
//
// One wavefront owns a tile of 64 consecutive samples of `sample_order` (key order when the
// caller provides it).  Inside a tile, samples with the same cell key form a run; the run's
// 3 x 3 pillar walk (9 binary searches on the sorted keys) is done once by lanes 0..8, the
// candidate points of the 9 ranges are then spread over the 64 lanes (coalesced reads of the
// sorted xyz array) and every sample of the run is tested against them in turn: one ballot
// per (sample, 64 candidates).  The fill pass repeats the walk and writes each sample's hits
// as one contiguous, rank-ordered store, so no atomics are used and the output is deterministic.
#include "common.h"

// fp32 expressions in this file must round exactly as written (no fused multiply-add).
#pragma clang fp contract(off)

#define NB_THREADS 256

struct NbArgs {
    const float *pts;          // sorted points [n,3]
    const int64_t *pt_keys;    // sorted keys [n]
    int64_t n;
    const float *samples;      // [m,3]
    const int64_t *sample_keys;
    int64_t m;
    const int32_t *order;      // nullable
    const int32_t *grid_ds;    // [num_pillars,2]
    int64_t num_pillars;
    const int32_t *cell_table; // nullable: [total_cells + 1] first sorted index of every cell
    int64_t total_cells;
    const int32_t *num_cells;  // [3]
    const float *radii;        // [3]
    int max_neighbors;
    int32_t *counts;           // raw hit counts per sample (written by COUNT, read by FILL)
    const int32_t *ends;       // FILL: inclusive running totals
    const int32_t *remap;      // FILL: nullable
    int64_t t;                 // FILL: number of output pairs
    int32_t *neigh;            // FILL: [t,2]
};

template <bool FILL, bool CAPPED>
__global__ void __launch_bounds__(NB_THREADS)
neighbors_kernel(NbArgs a)
{
    const int lane = pccnn_lane();
    const int64_t wave = ((int64_t)blockIdx.x * NB_THREADS + threadIdx.x) >> 6;
    const int64_t base = wave * 64;
    if (base >= a.m) return;                                   // wave-uniform
    const int nvalid = (int)((a.m - base) < 64 ? (a.m - base) : 64);
    const bool valid = lane < nvalid;

    int s = 0;
    long long key = -1;
    float sx = 0.f, sy = 0.f, sz = 0.f;
    if (valid) {
        s = a.order ? a.order[base + lane] : (int)(base + lane);
        key = a.sample_keys[s];
        sx = a.samples[(int64_t)s * 3 + 0];
        sy = a.samples[(int64_t)s * 3 + 1];
        sz = a.samples[(int64_t)s * 3 + 2];
    }
    const int nc0 = a.num_cells[0], nc1 = a.num_cells[1], nc2 = a.num_cells[2];
    const float ir0 = __fdiv_rn(1.0f, a.radii[0]);
    const float ir1 = __fdiv_rn(1.0f, a.radii[1]);
    const float ir2 = __fdiv_rn(1.0f, a.radii[2]);

    int key_lo = (int)(key & 0xffffffffll), key_hi = (int)(key >> 32);
    int prev_lo = __shfl_up(key_lo, 1), prev_hi = __shfl_up(key_hi, 1);
    const bool head = valid && (lane == 0 || prev_lo != key_lo || prev_hi != key_hi);
    unsigned long long headmask = __ballot(head);

    int my_cnt = 0;                                            // hits seen so far for this lane's sample
    int my_off = 0, my_raw = 0;                                // FILL: first output slot / uncapped hit count
    if (FILL && valid) {
        my_off = s > 0 ? a.ends[s - 1] : 0;
        if (CAPPED) my_raw = a.counts[s];
    }
    const unsigned long long lt = pccnn_lanemask_lt();

    while (headmask) {
        const int h = __builtin_ctzll(headmask);
        headmask &= headmask - 1;
        const int e = __builtin_amdgcn_readfirstlane(headmask ? __builtin_ctzll(headmask) : nvalid);
        const long long runkey = pccnn_bcast_ll(key, h);

        // key -> (batch, c0, c1, c2); 32-bit arithmetic whenever the key allows it
        long long pil;                                         // (batch * nc0 + c0) * nc1 + c1
        int c0, c1, c2;
        if (runkey >= 0 && runkey < 0x7fffffffll) {
            unsigned int k = (unsigned int)runkey;
            c2 = (int)(k % (unsigned int)nc2); k /= (unsigned int)nc2;
            c1 = (int)(k % (unsigned int)nc1); pil = k; k /= (unsigned int)nc1;
            c0 = (int)(k % (unsigned int)nc0);
        } else {
            long long k = runkey;
            c2 = (int)(k % nc2); k /= nc2;
            c1 = (int)(k % nc1); pil = k; k /= nc1;
            c0 = (int)(k % nc0);
        }

        int first = 0, len = 0;
        if (lane < 9 && runkey >= 0) {
            const int dx = lane / 3 - 1, dy = lane % 3 - 1;
            const int x = c0 + dx, y = c1 + dy;
            if (x >= 0 && x < nc0 && y >= 0 && y < nc1) {
                const long long pillar = pil + (long long)dx * nc1 + dy;
                const int cmin = c2 > 0 ? c2 - 1 : 0, cmax = c2 + 1 < nc2 ? c2 + 1 : nc2 - 1;
                if (a.cell_table) {
                    // cells cmin..cmax of the pillar are consecutive keys: two table reads give their range
                    const long long kbase = pillar * nc2;
                    if (pillar >= 0 && kbase + cmax + 1 <= a.total_cells) {
                        first = a.cell_table[kbase + cmin];
                        len = a.cell_table[kbase + cmax + 1] - first;
                        if (first < 0 || len < 0 || (int64_t)first + len > a.n) len = 0;
                    }
                } else if (pillar >= 0 && pillar < a.num_pillars) {
                    int lo = a.grid_ds[2 * pillar], hi = a.grid_ds[2 * pillar + 1];
                    lo = lo < 0 ? 0 : lo;
                    hi = hi > a.n ? (int)a.n : hi;
                    if (hi > lo) {
                        // keys of the cells c2-1 .. c2+1 of this pillar
                        const long long kbase = pillar * nc2;
                        const long long kmin = kbase + cmin;
                        const long long kmax = kbase + cmax;
                        int lb = lo, ub = hi;
                        while (lb < ub) {
                            int mid = (lb + ub) >> 1;
                            if (a.pt_keys[mid] < kmin) lb = mid + 1; else ub = mid;
                        }
                        first = lb;
                        ub = hi;
                        while (lb < ub) {
                            int mid = (lb + ub) >> 1;
                            if (a.pt_keys[mid] <= kmax) lb = mid + 1; else ub = mid;
                        }
                        len = lb - first;
                    }
                }
            }
        }
        int st[9], ln[9], total = 0;
#pragma unroll
        for (int o = 0; o < 9; ++o) {
            st[o] = __builtin_amdgcn_readlane(first, o);
            ln[o] = __builtin_amdgcn_readlane(len, o);
            total += ln[o];
        }

        for (int cb = 0; cb < total; cb += 64) {
            const int j = cb + lane;
            const bool cvalid = j < total;
            int idx = 0, rem = j;
#pragma unroll
            for (int o = 0; o < 9; ++o) {
                if (rem >= 0 && rem < ln[o]) idx = st[o] + rem;
                rem -= ln[o];
            }
            float px = 0.f, py = 0.f, pz = 0.f;
            if (cvalid) {
                px = a.pts[(int64_t)idx * 3 + 0];
                py = a.pts[(int64_t)idx * 3 + 1];
                pz = a.pts[(int64_t)idx * 3 + 2];
            }
            int out_id = idx;
            if (FILL && cvalid && a.remap) out_id = a.remap[idx];

            for (int q = h; q < e; ++q) {
                const float qx = pccnn_bcast_f(sx, q), qy = pccnn_bcast_f(sy, q), qz = pccnn_bcast_f(sz, q);
                // fp32, no contraction: ((s - p) * (1/r)) squared, summed x, y, z; the reference tests
                // sqrt(acc) < 1, which for a correctly rounded fp32 sqrt holds exactly when acc < 1
                // (the largest float below 1 has a root below the midpoint to 1, so it rounds down).
                const float vx = (qx - px) * ir0;
                const float vy = (qy - py) * ir1;
                const float vz = (qz - pz) * ir2;
                const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                const bool hit = cvalid && (acc < 1.0f);
                const unsigned long long bal = __ballot(hit);
                const int c = __popcll(bal);
                if (FILL) {
                    // my_off + my_cnt of lane q = next free slot of that sample (uncapped case)
                    const int qoff = pccnn_bcast_i(CAPPED ? my_off : my_off + my_cnt, q);
                    const int qs = pccnn_bcast_i(s, q);
                    if (hit) {
                        int slot = __popcll(bal & lt);
                        bool take = true;
                        if (CAPPED) {
                            const int qraw = pccnn_bcast_i(my_raw, q);
                            const int r = pccnn_bcast_i(my_cnt, q) + slot;
                            slot = r;
                            if (qraw > a.max_neighbors) {
                                slot = (int)(((long long)r * a.max_neighbors) / qraw);
                                take = (int)(((long long)(r + 1) * a.max_neighbors) / qraw) > slot;
                            }
                        }
                        const int64_t pos = (int64_t)qoff + slot;
                        if (take && pos < a.t) {
                            int2 pr;
                            pr.x = out_id;
                            pr.y = qs;
                            ((int2 *)a.neigh)[pos] = pr;
                        }
                    }
                }
                if (lane == q) my_cnt += c;
            }
        }
    }
    if (!FILL && valid) a.counts[s] = my_cnt;
}

// table[c] = index of the first sorted point whose key is >= c, for c in [0, total_cells].  The lane of
// every point that starts a new key owns the entries between the previous key and its own (lane n owns
// the tail); the 64 lanes of a wavefront then fill each other's gaps together, so a long run of empty
// cells is written as coalesced stores instead of by a single thread.
__global__ void __launch_bounds__(256)
cell_table_kernel(const int64_t *__restrict__ keys, int64_t n, int64_t total_cells, int32_t *__restrict__ table)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    long long from = 0, to = -1;                                    // table[from..to] = i (empty when to < from)
    if (i == n) {
        from = (n > 0 ? keys[n - 1] + 1 : 0);
        to = total_cells;
    } else if (i < n) {
        const long long key = keys[i];
        const long long prev = i > 0 ? keys[i - 1] : -1;
        if (key != prev) { from = prev + 1; to = key; }
    }
    if (from < 0) from = 0;
    if (to > total_cells) to = total_cells;
    const int lane = pccnn_lane();
    unsigned long long todo = __ballot(to >= from);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const long long f = pccnn_bcast_ll(from, src), t = pccnn_bcast_ll(to, src);
        const int32_t v = (int32_t)pccnn_bcast_ll((long long)i, src);
        for (long long c = f + lane; c <= t; c += 64) table[c] = v;
    }
}

extern "C" int pccnn_build_cell_table(const int64_t *sorted_keys, int64_t n, int64_t total_cells,
                                      int32_t *cell_table_out, void *stream)
{
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31) && total_cells > 0 && total_cells < (1ll << 40), PCCNN_ERR_INVALID,
                  "pccnn_build_cell_table: n=%lld total_cells=%lld", (long long)n, (long long)total_cells);
    PCCNN_REQUIRE(cell_table_out && (n == 0 || sorted_keys), PCCNN_ERR_INVALID, "pccnn_build_cell_table: null pointer");
    PccnnTimed timed(PCCNN_T_GRID, (hipStream_t)stream);
    cell_table_kernel<<<(unsigned)pccnn_ceil_div(n + 1, 256), 256, 0, (hipStream_t)stream>>>(sorted_keys, n, total_cells,
                                                                                          cell_table_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

extern "C" size_t pccnn_find_neighbors_workspace_bytes(int64_t m)
{
    if (m < 1) m = 1;
    return pccnn_align((size_t)m * sizeof(int32_t)) + pccnn_align(pccnn_scan_tmp_elems(m) * sizeof(int32_t)) + 256;
}

static int nb_validate(const char *who, const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                       const float *samples, const int64_t *sample_keys, int64_t m, const int32_t *grid_ds,
                       int64_t num_pillars, const int32_t *cell_table, int64_t total_cells, const int32_t *num_cells, const float *radii, int d, int max_neighbors, void *workspace,
                       size_t workspace_bytes)
{
    PCCNN_REQUIRE(d == 3, PCCNN_ERR_UNSUPPORTED, "%s: d=%d is not supported (d must be 3)", who, d);
    PCCNN_REQUIRE(n >= 0 && m >= 0 && n < (1ll << 31) && m < (1ll << 31), PCCNN_ERR_INVALID, "%s: n=%lld m=%lld",
                  who, (long long)n, (long long)m);
    PCCNN_REQUIRE(max_neighbors >= 0, PCCNN_ERR_INVALID, "%s: max_neighbors=%d", who, max_neighbors);
    PCCNN_REQUIRE(num_pillars > 0, PCCNN_ERR_INVALID, "%s: num_pillars=%lld", who, (long long)num_pillars);
    PCCNN_REQUIRE(cell_table == nullptr || total_cells > 0, PCCNN_ERR_INVALID, "%s: cell_table with total_cells=%lld",
                  who, (long long)total_cells);
    PCCNN_REQUIRE(grid_ds && num_cells && radii, PCCNN_ERR_INVALID, "%s: null grid pointer", who);
    PCCNN_REQUIRE(n == 0 || (pts_sorted && pt_keys_sorted), PCCNN_ERR_INVALID, "%s: null point pointer", who);
    PCCNN_REQUIRE(m == 0 || (samples && sample_keys), PCCNN_ERR_INVALID, "%s: null sample pointer", who);
    PCCNN_REQUIRE(workspace && workspace_bytes >= pccnn_find_neighbors_workspace_bytes(m), PCCNN_ERR_WORKSPACE,
                  "%s: workspace of %zu bytes, need %zu", who, workspace_bytes,
                  pccnn_find_neighbors_workspace_bytes(m));
    return PCCNN_OK;
}

extern "C" int pccnn_find_neighbors_count(const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                                          const float *samples, const int64_t *sample_keys, int64_t m,
                                          const int32_t *sample_order, const int32_t *grid_ds,
                                          int64_t num_pillars, const int32_t *cell_table, int64_t total_cells,
                                          const int32_t *num_cells, const float *radii, int d, int max_neighbors,
                                          int32_t *ends_out, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = nb_validate("pccnn_find_neighbors_count", pts_sorted, pt_keys_sorted, n, samples, sample_keys, m, grid_ds,
                         num_pillars, cell_table, total_cells, num_cells, radii, d, max_neighbors, workspace,
                         workspace_bytes);
    if (rc != PCCNN_OK) return rc;
    if (m == 0) return PCCNN_OK;
    PCCNN_REQUIRE(ends_out, PCCNN_ERR_INVALID, "pccnn_find_neighbors_count: null ends_out");
    hipStream_t s = (hipStream_t)stream;
    PccnnArena arena(workspace, workspace_bytes);
    int32_t *counts = arena.take<int32_t>((size_t)m);
    int32_t *scan_tmp = arena.take<int32_t>(pccnn_scan_tmp_elems(m));
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_find_neighbors_count: workspace too small");
    NbArgs a;
    a.pts = pts_sorted; a.pt_keys = pt_keys_sorted; a.n = n;
    a.samples = samples; a.sample_keys = sample_keys; a.m = m;
    a.order = sample_order; a.grid_ds = grid_ds; a.num_pillars = num_pillars;
    a.cell_table = cell_table; a.total_cells = total_cells;
    a.num_cells = num_cells; a.radii = radii; a.max_neighbors = max_neighbors;
    a.counts = counts; a.ends = nullptr; a.remap = nullptr; a.t = 0; a.neigh = nullptr;
    int64_t waves = pccnn_ceil_div(m, 64);
    {
        PccnnTimed timed(PCCNN_T_NB_COUNT, s);
        neighbors_kernel<false, false><<<(unsigned)pccnn_ceil_div(waves, NB_THREADS / 64), NB_THREADS, 0, s>>>(a);
    }
    PCCNN_LAUNCH_CHECK();
    PccnnTimed timed(PCCNN_T_SCAN, s);
    return pccnn_scan_inclusive_i32(counts, ends_out, m, max_neighbors, scan_tmp, s);
}

extern "C" int pccnn_find_neighbors_fill(const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                                         const float *samples, const int64_t *sample_keys, int64_t m,
                                         const int32_t *sample_order, const int32_t *grid_ds,
                                         int64_t num_pillars, const int32_t *cell_table, int64_t total_cells,
                                          const int32_t *num_cells, const float *radii, int d, int max_neighbors,
                                         const int32_t *ends, const int32_t *point_remap, int64_t t,
                                         int32_t *neigh_out, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = nb_validate("pccnn_find_neighbors_fill", pts_sorted, pt_keys_sorted, n, samples, sample_keys, m, grid_ds,
                         num_pillars, cell_table, total_cells, num_cells, radii, d, max_neighbors, workspace,
                         workspace_bytes);
    if (rc != PCCNN_OK) return rc;
    PCCNN_REQUIRE(t >= 0 && t < (1ll << 31), PCCNN_ERR_INVALID, "pccnn_find_neighbors_fill: t=%lld", (long long)t);
    if (m == 0 || t == 0) return PCCNN_OK;
    PCCNN_REQUIRE(ends && neigh_out, PCCNN_ERR_INVALID, "pccnn_find_neighbors_fill: null pointer");
    hipStream_t s = (hipStream_t)stream;
    PccnnArena arena(workspace, workspace_bytes);
    int32_t *counts = arena.take<int32_t>((size_t)m);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_find_neighbors_fill: workspace too small");
    NbArgs a;
    a.pts = pts_sorted; a.pt_keys = pt_keys_sorted; a.n = n;
    a.samples = samples; a.sample_keys = sample_keys; a.m = m;
    a.order = sample_order; a.grid_ds = grid_ds; a.num_pillars = num_pillars;
    a.cell_table = cell_table; a.total_cells = total_cells;
    a.num_cells = num_cells; a.radii = radii; a.max_neighbors = max_neighbors;
    a.counts = counts; a.ends = ends; a.remap = point_remap; a.t = t; a.neigh = neigh_out;
    int64_t waves = pccnn_ceil_div(m, 64);
    {
        PccnnTimed timed(PCCNN_T_NB_FILL, s);
        if (max_neighbors > 0)
            neighbors_kernel<true, true><<<(unsigned)pccnn_ceil_div(waves, NB_THREADS / 64), NB_THREADS, 0, s>>>(a);
        else
            neighbors_kernel<true, false><<<(unsigned)pccnn_ceil_div(waves, NB_THREADS / 64), NB_THREADS, 0, s>>>(a);
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}
