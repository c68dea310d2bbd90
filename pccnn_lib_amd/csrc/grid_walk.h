// The pillar grid as the kernels that walk it see it: the pillar table [num_pillars, 2] of index ranges into the
// sorted points, and, when the grid is small enough to afford one, the per-cell start table.
#pragma once
#include "common.h"

struct GridRef {
    const int32_t *cell_table;   // nullable: [total_cells + 1] first sorted index of every cell
    int64_t total_cells;
    const int32_t *grid_ds;      // [num_pillars, 2]
    int64_t num_pillars;
    const int64_t *pt_keys;      // sorted keys [n]
    int64_t n;
};

#ifdef __HIPCC__
// Index range [first, first + len) of the sorted points that lie in cells cmin..cmax of `pillar`.
__device__ __forceinline__ void grid_pillar_range(const GridRef &a, long long pillar, int nc2, int cmin, int cmax,
                                                int &first, int &len)
{
    first = 0;
    len = 0;
    const long long kbase = pillar * nc2;
    if (a.cell_table) {
        // cells cmin..cmax of the pillar are consecutive keys: two table reads give their range
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

#endif
