// Bounding box, cell keys and the pillar table.  All three are HBM-streaming kernels:
// one thread per point, coalesced reads of the xyz / key arrays.
#include "common.h"

// fp32 expressions in this file must round exactly as written (no fused multiply-add).
#pragma clang fp contract(off)

// ----------------------------------------------------------- bounding box

__device__ __forceinline__ void atomic_min_f32(float *addr, float v)
{
    // Order-preserving integer views of IEEE floats: non-negative values compare as signed
    // ints, negative values compare reversed as unsigned ints.
    if (v >= 0.0f) atomicMin((int *)addr, __float_as_int(v));
    else atomicMax((unsigned int *)addr, __float_as_uint(v));
}
__device__ __forceinline__ void atomic_max_f32(float *addr, float v)
{
    if (v >= 0.0f) atomicMax((int *)addr, __float_as_int(v));
    else atomicMin((unsigned int *)addr, __float_as_uint(v));
}

__global__ void bbox_init_kernel(float *mn, float *mx, int count)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) { mn[i] = __int_as_float(0x7f800000); mx[i] = __int_as_float(0xff800000); }
}

// The boxes the lanes of a wavefront hold (cloud `cur`, or none when cur < 0) go to memory: for every distinct
// cloud among them, the lanes holding it are reduced with lane exchanges and one lane issues the
// atomics.  All lanes of the wavefront must call this together.
template <int D>
__device__ __forceinline__ void bbox_flush_wave(int cur, const float (&lo)[D], const float (&hi)[D], float *mn,
                                                float *mx)
{
    const float inf = __int_as_float(0x7f800000);
    unsigned long long todo = __ballot(cur >= 0);
    while (todo != 0ull) {
        const int b = pccnn_bcast_i(cur, __builtin_ctzll(todo));
        const bool mine = cur == b;
#pragma unroll
        for (int k = 0; k < D; ++k) {
            const float l = pccnn_wave_minmax<false>(mine ? lo[k] : inf);
            const float h = pccnn_wave_minmax<true>(mine ? hi[k] : -inf);
            if (pccnn_lane() == 0) {
                atomic_min_f32(&mn[b * D + k], l);
                atomic_max_f32(&mx[b * D + k], h);
            }
        }
        todo &= ~__ballot(mine);
    }
}

// Chunked reduction.  A workgroup owns one contiguous chunk of the point list and every thread keeps a running box
// for the cloud it is currently in (clouds are normally stored one after the other).  When some lane of a
// wavefront meets another cloud, the wavefront flushes what it holds, one set of atomics per distinct cloud; at the
// end a wavefront whose lanes all hold the same cloud reduces with exchanges, and a workgroup whose four
// wavefronts agree combines them in LDS, so a launch issues a few hundred atomics per box corner at most.
template <int D>
__global__ void __launch_bounds__(256)
bbox_reduce_kernel(const float *__restrict__ pts, const int32_t *__restrict__ batch_ids, int64_t n, int batch_size,
                   float *mn, float *mx, PccnnBoxMask mask)
{
    __shared__ float lds_lo[4][D], lds_hi[4][D];
    __shared__ int lds_b[4];
    const float inf = __int_as_float(0x7f800000);
    int cur = -1;
    float lo[D], hi[D];
#pragma unroll
    for (int k = 0; k < D; ++k) { lo[k] = inf; hi[k] = -inf; }
    const int64_t chunk = (n + gridDim.x - 1) / gridDim.x;
    const int64_t chunk_end = ((int64_t)blockIdx.x + 1) * chunk < n ? ((int64_t)blockIdx.x + 1) * chunk : n;
    // four points per thread in flight: their loads do not depend on each other, the box update does; the trip
    // count is the same for all threads of the workgroup, so the wavefront-wide flush sits in uniform control flow
    constexpr int UNROLL = 4;
    for (int64_t w0 = (int64_t)blockIdx.x * chunk; w0 < chunk_end; w0 += (int64_t)UNROLL * blockDim.x) {
        int bs[UNROLL];
        float vs[UNROLL][D];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t i = w0 + (int64_t)u * blockDim.x + threadIdx.x;
            bs[u] = -1;
            if (i < chunk_end) {
                const int b = mask.cloud_of(batch_ids, i);
                bs[u] = (b >= 0 && b < batch_size) ? b : -1;          // ids outside the table are ignored
#pragma unroll
                for (int k = 0; k < D; ++k) vs[u][k] = pts[i * D + k];
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int b = bs[u];
            if (__any(b >= 0 && cur >= 0 && b != cur)) {
                bbox_flush_wave<D>(cur, lo, hi, mn, mx);
                cur = -1;
#pragma unroll
                for (int k = 0; k < D; ++k) { lo[k] = inf; hi[k] = -inf; }
            }
            if (b >= 0) {
                cur = b;
#pragma unroll
                for (int k = 0; k < D; ++k) {
                    lo[k] = fminf(lo[k], vs[u][k]);
                    hi[k] = fmaxf(hi[k], vs[u][k]);
                }
            }
        }
    }
    const int lane = pccnn_lane(), wave = threadIdx.x >> 6;
    const unsigned long long have = __ballot(cur >= 0);
    const int b0 = have ? pccnn_bcast_i(cur, __builtin_ctzll(have)) : -1;
    const bool wave_uniform = __ballot(cur >= 0 && cur != b0) == 0ull;     // idle lanes hold the neutral box
    if (wave_uniform) {
#pragma unroll
        for (int k = 0; k < D; ++k) {
            lo[k] = pccnn_wave_minmax<false>(lo[k]);
            hi[k] = pccnn_wave_minmax<true>(hi[k]);
        }
        if (lane == 0) {
            lds_b[wave] = b0;
#pragma unroll
            for (int k = 0; k < D; ++k) { lds_lo[wave][k] = lo[k]; lds_hi[wave][k] = hi[k]; }
        }
    } else {
        if (lane == 0) lds_b[wave] = -2;                              // flushed here, cloud by cloud
        bbox_flush_wave<D>(cur, lo, hi, mn, mx);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const bool same = lds_b[0] == lds_b[1] && lds_b[0] == lds_b[2] && lds_b[0] == lds_b[3];
        for (int w = 0; w < 4; ++w) {
            const int b = lds_b[w];
            if (b < 0) continue;
            if (same && w > 0) break;
            for (int k = 0; k < D; ++k) {
                float l = lds_lo[w][k], h = lds_hi[w][k];
                if (same)
                    for (int w2 = 1; w2 < 4; ++w2) { l = fminf(l, lds_lo[w2][k]); h = fmaxf(h, lds_hi[w2][k]); }
                atomic_min_f32(&mn[b * D + k], l);
                atomic_max_f32(&mx[b * D + k], h);
            }
        }
    }
}

__global__ void bbox_pad_kernel(float *mn, float *mx, int count, PccnnBoxMask mask)
{
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) {
        const float l = mn[i] - 1e-6f, h = mx[i] + 1e-6f;
        mn[i] = l; mx[i] = h;
        mask.second_copy(i, count, l, h);
    }
    if (mask.tail != nullptr) {
        // (the word is behind all the box values only when this is the launch's one workgroup)
        __threadfence_system();
        __syncthreads();
        if (i == 0) mask.publish(count);
    }
}

// A small cloud (up to BBOX_SMALL_POINTS points, up to BBOX_SMALL_CLOUDS clouds): one workgroup, the boxes in LDS,
// initial values, reduction and padding in one launch instead of three.  Same minima and maxima (they do not depend
// on the order of the comparisons), same padding.
#define BBOX_SMALL_POINTS 16384
#define BBOX_SMALL_CLOUDS 64
template <int D>
__global__ void __launch_bounds__(1024)
bbox_small_kernel(const float *__restrict__ pts, const int32_t *__restrict__ batch_ids, int64_t n, int batch_size,
                  float *__restrict__ mn, float *__restrict__ mx, PccnnBoxMask mask)
{
    __shared__ float box_lo[BBOX_SMALL_CLOUDS * D], box_hi[BBOX_SMALL_CLOUDS * D];
    const float inf = __int_as_float(0x7f800000);
    const int count = batch_size * D;
    for (int i = threadIdx.x; i < count; i += blockDim.x) { box_lo[i] = inf; box_hi[i] = -inf; }
    __syncthreads();
    int cur = -1;
    float lo[D], hi[D];
#pragma unroll
    for (int k = 0; k < D; ++k) { lo[k] = inf; hi[k] = -inf; }
    // the same trip count for every thread: the wavefront-wide flush sits in uniform control flow
    for (int64_t w0 = 0; w0 < n; w0 += blockDim.x) {
        const int64_t i = w0 + threadIdx.x;
        int b = -1;
        float v[D];
        if (i < n) {
            b = mask.cloud_of(batch_ids, i);
            if (b < 0 || b >= batch_size) b = -1;                      // ids outside the table are ignored
#pragma unroll
            for (int k = 0; k < D; ++k) v[k] = pts[i * D + k];
        }
        if (__any(b >= 0 && cur >= 0 && b != cur)) {
            bbox_flush_wave<D>(cur, lo, hi, box_lo, box_hi);
            cur = -1;
#pragma unroll
            for (int k = 0; k < D; ++k) { lo[k] = inf; hi[k] = -inf; }
        }
        if (b >= 0) {
            cur = b;
#pragma unroll
            for (int k = 0; k < D; ++k) { lo[k] = fminf(lo[k], v[k]); hi[k] = fmaxf(hi[k], v[k]); }
        }
    }
    bbox_flush_wave<D>(cur, lo, hi, box_lo, box_hi);
    __syncthreads();
    for (int i = threadIdx.x; i < count; i += blockDim.x) {
        const float l = box_lo[i] - 1e-6f, h = box_hi[i] + 1e-6f;
        mn[i] = l; mx[i] = h;
        mask.second_copy(i, count, l, h);
    }
    if (mask.tail != nullptr) {
        __threadfence_system();
        __syncthreads();
        if (threadIdx.x == 0) mask.publish(count);
    }
}

extern "C" int pccnn_bounding_box(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                                  float *aabb_min_out, float *aabb_max_out, void *stream)
{
    return pccnn_bounding_box_masked(pts, batch_ids, n, d, batch_size, aabb_min_out, aabb_max_out, PccnnBoxMask{},
                                     stream);
}

int pccnn_bounding_box_masked(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                              float *aabb_min_out, float *aabb_max_out, const PccnnBoxMask &mask, void *stream)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_bounding_box: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(n >= 0 && batch_size > 0, PCCNN_ERR_INVALID, "pccnn_bounding_box: n=%lld batch_size=%d",
                  (long long)n, batch_size);
    PCCNN_REQUIRE(aabb_min_out && aabb_max_out && (n == 0 || (pts && batch_ids)), PCCNN_ERR_INVALID,
                  "pccnn_bounding_box: null pointer");
    hipStream_t s = (hipStream_t)stream;
    int count = batch_size * d;
    if (n > 0 && n <= BBOX_SMALL_POINTS && batch_size <= BBOX_SMALL_CLOUDS) {
        PCCNN_DIM_DISPATCH(d, bbox_small_kernel, <<<1, 1024, 0, s>>>(pts, batch_ids, n, batch_size, aabb_min_out,
                                                                    aabb_max_out, mask));
        PCCNN_LAUNCH_CHECK();
        return PCCNN_OK;
    }
    bbox_init_kernel<<<(unsigned)pccnn_ceil_div(count, 256), 256, 0, s>>>(aabb_min_out, aabb_max_out, count);
    PCCNN_LAUNCH_CHECK();
    if (n > 0) {
        // every workgroup ends with a handful of integer atomics per box corner, and with one cloud they all meet on
        // the same six addresses: few workgroups, each with four points per thread in flight
        int64_t blocks = pccnn_ceil_div(n, 256 * 4);
        if (blocks > 256) blocks = 256;
        PCCNN_DIM_DISPATCH(d, bbox_reduce_kernel, <<<(unsigned)blocks, 256, 0, s>>>(pts, batch_ids, n, batch_size,
                                                                                    aabb_min_out, aabb_max_out, mask));
        PCCNN_LAUNCH_CHECK();
    }
    bbox_pad_kernel<<<(unsigned)pccnn_ceil_div(count, 256), 256, 0, s>>>(aabb_min_out, aabb_max_out, count, mask);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// num_cells[k] = max_b int((max[b][k] - min[b][k]) / cell[k]) + 1: one thread per dimension, clouds in order.
__global__ void num_cells_kernel(const float *__restrict__ mn, const float *__restrict__ mx,
                                 const float *__restrict__ cell, int batch_size, int d, int32_t *__restrict__ out)
{
    const int k = threadIdx.x;
    if (k >= d) return;
    int best = 0;
    for (int b = 0; b < batch_size; ++b) {
        const int c = (int)__fdiv_rn(mx[b * d + k] - mn[b * d + k], cell[k]) + 1;
        best = (b == 0 || c > best) ? c : best;
    }
    out[k] = best;
}

extern "C" int pccnn_num_cells(const float *aabb_min, const float *aabb_max, const float *cell_size, int batch_size,
                               int d, int32_t *num_cells_out, void *stream)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED, "pccnn_num_cells: d=%d is not supported (2 <= d <= 6)",
                  d);
    PCCNN_REQUIRE(batch_size > 0, PCCNN_ERR_INVALID, "pccnn_num_cells: batch_size=%d", batch_size);
    PCCNN_REQUIRE(aabb_min && aabb_max && cell_size && num_cells_out, PCCNN_ERR_INVALID, "pccnn_num_cells: null pointer");
    num_cells_kernel<<<1, 64, 0, (hipStream_t)stream>>>(aabb_min, aabb_max, cell_size, batch_size, d, num_cells_out);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// ------------------------------------------------------------------- keys

// SIZED: the grid size arrives by value (`sized`), and the first workgroup also writes it to num_cells_out, where the
// kernels after this one read it; otherwise it is read from num_cells.
template <int D, bool SIZED>
__global__ void __launch_bounds__(256)
compute_keys_kernel(const float *__restrict__ pts, const int32_t *__restrict__ batch_ids,
                    const float *__restrict__ aabb_min, const int32_t *__restrict__ num_cells,
                    const float *__restrict__ cell_size, int64_t n, int64_t *__restrict__ keys, PccnnGridDims sized,
                    int32_t *__restrict__ num_cells_out)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (SIZED && blockIdx.x == 0 && threadIdx.x < D) num_cells_out[threadIdx.x] = sized.v[threadIdx.x];
    if (i >= n) return;
    int b = batch_ids[i];
    long long key = 0, accum = 1;
#pragma unroll
    for (int k = D - 1; k >= 0; --k) {
        // fp32, exactly in this order: subtract the box corner, multiply by the fp32
        // reciprocal of the cell size, floor, clamp.
        float inv = __fdiv_rn(1.0f, cell_size[k]);
        float rel = (pts[i * D + k] - aabb_min[(int64_t)b * D + k]) * inv;
        int nc = SIZED ? sized.v[k] : num_cells[k];
        int c = (int)floorf(rel);
        c = max(0, min(c, nc - 1));
        key += (long long)c * accum;
        accum *= nc;
    }
    keys[i] = key + accum * (long long)b;
}

extern "C" int pccnn_compute_keys(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                                  const int32_t *num_cells, const float *cell_size, int64_t n, int d,
                                  int64_t *keys_out, void *stream)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_compute_keys: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(n >= 0, PCCNN_ERR_INVALID, "pccnn_compute_keys: n=%lld", (long long)n);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(pts && batch_ids && aabb_min && num_cells && cell_size && keys_out, PCCNN_ERR_INVALID,
                  "pccnn_compute_keys: null pointer");
    PccnnTimed timed(PCCNN_T_KEYS, (hipStream_t)stream);
    const unsigned blocks = (unsigned)pccnn_ceil_div(n, 256);
    hipStream_t s = (hipStream_t)stream;
    const PccnnGridDims none = {};
#define KEYS_GO(D) compute_keys_kernel<D, false><<<blocks, 256, 0, s>>>(pts, batch_ids, aabb_min, num_cells, cell_size, n, \
                                                                       (int64_t *)keys_out, none, nullptr)
    switch (d) {
    case 2: KEYS_GO(2); break;
    case 3: KEYS_GO(3); break;
    case 4: KEYS_GO(4); break;
    case 5: KEYS_GO(5); break;
    default: KEYS_GO(6); break;
    }
#undef KEYS_GO
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// pccnn_compute_keys for a grid size known on the host (d ints): the keys are computed from those numbers, and the
// same launch writes them to num_cells_out i32[d] on the device for the kernels that follow.
int pccnn_compute_keys_sized(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                             const int32_t *num_cells_host, const float *cell_size, int64_t n, int d,
                             int32_t *num_cells_out, int64_t *keys_out, hipStream_t s)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_compute_keys: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(n >= 0, PCCNN_ERR_INVALID, "pccnn_compute_keys: n=%lld", (long long)n);
    PCCNN_REQUIRE(num_cells_host && num_cells_out && cell_size && aabb_min && (n == 0 || (pts && batch_ids && keys_out)),
                  PCCNN_ERR_INVALID, "pccnn_compute_keys: null pointer");
    PccnnGridDims dims = {};
    for (int k = 0; k < d; ++k) dims.v[k] = num_cells_host[k];
    PccnnTimed timed(PCCNN_T_KEYS, s);
    const unsigned blocks = (unsigned)pccnn_ceil_div(n > 0 ? n : 1, 256);       // n == 0: the size is still written
#define KEYS_GO(D) compute_keys_kernel<D, true><<<blocks, 256, 0, s>>>(pts, batch_ids, aabb_min, nullptr, cell_size, n, \
                                                                      keys_out, dims, num_cells_out)
    switch (d) {
    case 2: KEYS_GO(2); break;
    case 3: KEYS_GO(3); break;
    case 4: KEYS_GO(4); break;
    case 5: KEYS_GO(5); break;
    default: KEYS_GO(6); break;
    }
#undef KEYS_GO
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// ------------------------------------------------------------ pillar grid

template <int D>
__global__ void __launch_bounds__(256)
build_grid_kernel(const int64_t *__restrict__ keys, int64_t n, const int32_t *__restrict__ num_cells,
                  int64_t num_pillars, int32_t *__restrict__ ds)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    long long div = 1;
#pragma unroll
    for (int k = 2; k < D; ++k) div *= num_cells[k];
    long long cur = keys[i] / div;
    if (cur < 0 || cur >= num_pillars) return;   // a key outside the table is never written
    long long prev = (i > 0) ? keys[i - 1] / div : -1;
    long long next = (i + 1 < n) ? keys[i + 1] / div : -1;
    if (i > 0 && prev != cur) ds[2 * cur] = (int32_t)i;
    if (i + 1 == n || next != cur) ds[2 * cur + 1] = (int32_t)(i + 1);
}

extern "C" int pccnn_build_grid_ds(const int64_t *sorted_keys, int64_t n, const int32_t *num_cells, int d,
                                   int64_t num_pillars, int32_t *grid_ds_out, void *stream)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_build_grid_ds: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(n >= 0 && num_pillars > 0 && num_pillars < (1ll << 30), PCCNN_ERR_INVALID,
                  "pccnn_build_grid_ds: n=%lld num_pillars=%lld", (long long)n, (long long)num_pillars);
    PCCNN_REQUIRE(grid_ds_out && num_cells && (n == 0 || sorted_keys), PCCNN_ERR_INVALID,
                  "pccnn_build_grid_ds: null pointer");
    hipStream_t s = (hipStream_t)stream;
    PccnnTimed timed(PCCNN_T_GRID, s);
    int rc = pccnn_fill_i32(grid_ds_out, 0, num_pillars * 2, s);
    if (rc != PCCNN_OK) return rc;
    if (n == 0) return PCCNN_OK;
    PCCNN_DIM_DISPATCH(d, build_grid_kernel, <<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, s>>>(sorted_keys, n, num_cells,
                                                                                          num_pillars, grid_ds_out));
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// Pillar table and per-cell table of a sorted key array in one launch (the results of pccnn_build_grid_ds, its zero
// fill included, and of pccnn_build_cell_table).  One lane per point plus one for the tail: the lane of a point that
// starts a new key owns the table entries between the previous key and its own, the lane of a point that starts a
// new pillar owns the empty pillars in between (they are zeroed) and writes the pillar's start, the pillar's last
// point writes its end; the lanes of a wavefront fill each other's runs together with coalesced stores.
template <int D, bool TABLE>
__global__ void __launch_bounds__(256)
grid_tables_kernel(const int64_t *__restrict__ keys, int64_t n, const int32_t *__restrict__ num_cells,
                   int64_t num_pillars, int64_t total_cells, int32_t *__restrict__ ds, int32_t *__restrict__ table)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    long long div = 1;
#pragma unroll
    for (int k = 2; k < D; ++k) div *= num_cells[k];
    long long from = 0, to = -1;                                    // table[from..to] = i (empty when to < from)
    long long zfrom = 0, zto = -1;                                  // pillars zfrom..zto are empty
    if (i == n) {
        const long long last = n > 0 ? keys[n - 1] : -1;
        from = last + 1;
        to = total_cells;
        zfrom = last >= 0 ? last / div + 1 : 0;
        zto = num_pillars - 1;
    } else if (i < n) {
        const long long key = keys[i];
        const long long prev = i > 0 ? keys[i - 1] : -1;
        if (key != prev) { from = prev + 1; to = key; }
        const long long cur = key / div;
        const long long prev_p = prev >= 0 ? prev / div : -1;
        const long long next_p = (i + 1 < n) ? keys[i + 1] / div : -1;
        if (cur >= 0 && cur < num_pillars) {                        // a key outside the table is never written
            if (prev_p != cur) ds[2 * cur] = (int32_t)i;
            if (i + 1 == n || next_p != cur) ds[2 * cur + 1] = (int32_t)(i + 1);
        }
        if (prev_p != cur) { zfrom = prev_p + 1; zto = cur - 1; }
    }
    if (zfrom < 0) zfrom = 0;
    if (zto > num_pillars - 1) zto = num_pillars - 1;
    const int lane = pccnn_lane();
    unsigned long long todo = __ballot(zto >= zfrom);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const long long f = pccnn_bcast_ll(zfrom, src) * 2, t = pccnn_bcast_ll(zto, src) * 2 + 1;
        for (long long c = f + lane; c <= t; c += 64) ds[c] = 0;
    }
    if (!TABLE) return;
    if (from < 0) from = 0;
    if (to > total_cells) to = total_cells;
    todo = __ballot(to >= from);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const long long f = pccnn_bcast_ll(from, src), t = pccnn_bcast_ll(to, src);
        const int32_t v = (int32_t)pccnn_bcast_ll((long long)i, src);
        for (long long c = f + lane; c <= t; c += 64) table[c] = v;
    }
}

static int grid_tables(const int64_t *sorted_keys, int64_t n, const int32_t *num_cells, int d, int64_t num_pillars,
                       int64_t total_cells, int32_t *grid_ds_out, int32_t *cell_table_out, hipStream_t s)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_grid_build: d=%d is not supported (2 <= d <= 6)", d);
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31) && num_pillars > 0 && num_pillars < (1ll << 30), PCCNN_ERR_INVALID,
                  "pccnn_grid_build: n=%lld num_pillars=%lld", (long long)n, (long long)num_pillars);
    PCCNN_REQUIRE(grid_ds_out && num_cells && (n == 0 || sorted_keys), PCCNN_ERR_INVALID,
                  "pccnn_grid_build: null pointer");
    PCCNN_REQUIRE(cell_table_out == nullptr || (total_cells > 0 && total_cells < (1ll << 40)), PCCNN_ERR_INVALID,
                  "pccnn_grid_build: total_cells=%lld", (long long)total_cells);
    PccnnTimed timed(PCCNN_T_GRID, s);
    const unsigned blocks = (unsigned)pccnn_ceil_div(n + 1, 256);
#define GRID_TABLES_GO(D)                                                                                        \
    do {                                                                                                         \
        if (cell_table_out != nullptr)                                                                           \
            grid_tables_kernel<D, true><<<blocks, 256, 0, s>>>(sorted_keys, n, num_cells, num_pillars, total_cells, \
                                                               grid_ds_out, cell_table_out);                     \
        else                                                                                                     \
            grid_tables_kernel<D, false><<<blocks, 256, 0, s>>>(sorted_keys, n, num_cells, num_pillars, 0,         \
                                                                grid_ds_out, nullptr);                           \
    } while (0)
    switch (d) {
    case 2: GRID_TABLES_GO(2); break;
    case 3: GRID_TABLES_GO(3); break;
    case 4: GRID_TABLES_GO(4); break;
    case 5: GRID_TABLES_GO(5); break;
    default: GRID_TABLES_GO(6); break;
    }
#undef GRID_TABLES_GO
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// ------------------------------------------------------------------- the four steps of a grid in one call
// Keys, stable sort (with the gather of the coordinates), pillar table and, when asked for, the per-cell start
// table: what Grid.compute_cell_ids + Grid.build_ds of the reference do (pccnn_lib/pc/Grid.py:40-72), as one entry
// point, so that a host layer pays one call instead of four.  The launches are those of the four entry points.
extern "C" size_t pccnn_grid_build_workspace_bytes(int64_t n) { return pccnn_sort_keys_workspace_bytes(n); }

extern "C" int pccnn_grid_build(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                                const int32_t *num_cells, const float *cell_size, int64_t n, int d, int key_bits,
                                int64_t num_pillars, int64_t total_cells, int64_t *keys_out, int64_t *sorted_keys_out,
                                int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out,
                                int32_t *cell_table_out, void *workspace, size_t workspace_bytes, void *stream)
{
    if (d == 3 && n > 0 && pts && batch_ids && aabb_min && num_cells && cell_size && keys_out && sorted_pts_out) {
        // three dimensions: the keys are computed by the sort's first histogram pass
        PccnnKeySource src = {pts, batch_ids, aabb_min, cell_size, num_cells, {}, nullptr, 0};
        int rc = pccnn_sort_keys_from_points(src, keys_out, n, key_bits, sorted_keys_out, perm_out, sorted_pts_out,
                                             workspace, workspace_bytes, stream);
        if (rc != PCCNN_OK) return rc;
        return grid_tables(sorted_keys_out, n, num_cells, d, num_pillars, total_cells, grid_ds_out, cell_table_out,
                           (hipStream_t)stream);
    }
    int rc = pccnn_compute_keys(pts, batch_ids, aabb_min, num_cells, cell_size, n, d, keys_out, stream);
    if (rc != PCCNN_OK) return rc;
    return pccnn_grid_build_from_keys(keys_out, pts, num_cells, n, d, key_bits, num_pillars, total_cells,
                                      sorted_keys_out, perm_out, sorted_pts_out, grid_ds_out, cell_table_out, workspace,
                                      workspace_bytes, stream);
}

// pccnn_grid_build for three dimensions and a grid size known on the host: the sort's first pass computes the keys
// from that size and writes the device copy.
int pccnn_grid_build_sized3(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                            const int32_t *num_cells_host, const float *cell_size, int64_t n, int key_bits,
                            int64_t num_pillars, int64_t total_cells, int32_t *num_cells_out, int64_t *keys_out,
                            int64_t *sorted_keys_out, int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out,
                            int32_t *cell_table_out, void *workspace, size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(n > 0 && num_cells_host && num_cells_out && keys_out && sorted_pts_out, PCCNN_ERR_INVALID,
                  "pccnn_grid_build_sized: null pointer or n=%lld", (long long)n);
    PccnnKeySource src = {pts, batch_ids, aabb_min, cell_size, nullptr, {}, num_cells_out, 1};
    for (int k = 0; k < 3; ++k) src.sized.v[k] = num_cells_host[k];
    int rc = pccnn_sort_keys_from_points(src, keys_out, n, key_bits, sorted_keys_out, perm_out, sorted_pts_out,
                                         workspace, workspace_bytes, stream);
    if (rc != PCCNN_OK) return rc;
    return grid_tables(sorted_keys_out, n, num_cells_out, 3, num_pillars, total_cells, grid_ds_out, cell_table_out,
                       (hipStream_t)stream);
}

int pccnn_grid_build_from_keys(const int64_t *keys, const float *pts, const int32_t *num_cells, int64_t n, int d,
                               int key_bits, int64_t num_pillars, int64_t total_cells, int64_t *sorted_keys_out,
                               int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out, int32_t *cell_table_out,
                               void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = pccnn_sort_keys(keys, n, key_bits, sorted_keys_out, perm_out, pts, d, sorted_pts_out, workspace,
                             workspace_bytes, stream);
    if (rc != PCCNN_OK) return rc;
    // pillar table and cell table from one launch
    return grid_tables(sorted_keys_out, n, num_cells, d, num_pillars, total_cells, grid_ds_out, cell_table_out,
                       (hipStream_t)stream);
}

