// Stable LSD radix sort of (64-bit cell key, 32-bit index) pairs, 8 bits per pass, only over
// the significant key bits.  Per pass:
//   1. radix_hist_kernel    : per-tile digit histogram staged in LDS, stored digit-major
//   2. radix_scan_kernel    : one workgroup per digit scans that digit's per-tile counts
//   3. radix_scatter_kernel : every tile re-reads its keys, ranks them with wave ballots
//                             (match-any on the digit bits), and scatters keys and indices;
//                             the last pass also gathers the xyz row of every point.
// Ties keep their input order in every pass, so the permutation is the stable argsort.
#include "common.h"

#define RS_THREADS 256
#define RS_MAX_ITEMS 8                                  // keys per thread and tile, at most
#define RS_WAVES (RS_THREADS / PCCNN_WAVE)

// Keys per thread of a tile: small inputs get small tiles, so that the launch still has a few hundred
// workgroups (a tile is walked in `items` rounds with barriers in between: few large tiles leave the chip
// idle), large inputs get the largest tiles (every tile pays a fixed set-up and a row of the histogram table).
static int rs_items_for(int64_t n)
{
    int64_t items = pccnn_ceil_div(n, (int64_t)RS_THREADS * 512);
    return (int)(items < 1 ? 1 : (items > RS_MAX_ITEMS ? RS_MAX_ITEMS : items));
}

__global__ void __launch_bounds__(RS_THREADS)
radix_hist_kernel(const int64_t *__restrict__ keys, int64_t n, int shift, int items, int32_t *__restrict__ tile_hist,
                  int64_t num_tiles)
{
    __shared__ int hist[256];
    hist[threadIdx.x] = 0;
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * RS_THREADS * items;
    for (int r = 0; r < items; ++r) {
        int64_t i = base + r * RS_THREADS + threadIdx.x;
        if (i < n) atomicAdd(&hist[(int)((keys[i] >> shift) & 0xff)], 1);
    }
    __syncthreads();
    tile_hist[(int64_t)threadIdx.x * num_tiles + blockIdx.x] = hist[threadIdx.x];
}

// One workgroup per digit: exclusive scan of that digit's per-tile counts (contiguous in the digit-major
// table), in place; the digit's total goes to digit_totals[digit].
__global__ void __launch_bounds__(256)
radix_scan_kernel(int32_t *__restrict__ tile_hist, int64_t num_tiles, int32_t *__restrict__ digit_totals)
{
    __shared__ int wave_tot[4];
    const int lane = pccnn_lane(), wave = threadIdx.x >> 6;
    int32_t *row = tile_hist + (int64_t)blockIdx.x * num_tiles;
    int carry = 0;
    for (int64_t base = 0; base < num_tiles; base += 256) {
        const int64_t i = base + threadIdx.x;
        const int x = i < num_tiles ? row[i] : 0;
        int incl = x;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int t = __shfl_up(incl, o);
            if (lane >= o) incl += t;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int add = carry, tot = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const int v = wave_tot[w];
            if (w < wave) add += v;
            tot += v;
        }
        if (i < num_tiles) row[i] = add + incl - x;
        carry += tot;
        __syncthreads();
    }
    if (threadIdx.x == 0) digit_totals[blockIdx.x] = carry;
}

template <bool FIRST, bool GATHER>
__global__ void __launch_bounds__(RS_THREADS)
radix_scatter_kernel(const int64_t *__restrict__ keys_in, const int32_t *__restrict__ vals_in, int64_t n, int shift,
                     int items, const int32_t *__restrict__ tile_offsets, int64_t num_tiles,
                     const int32_t *__restrict__ digit_totals, int64_t *__restrict__ keys_out, int32_t *__restrict__ vals_out,
                     const float *__restrict__ pts, float *__restrict__ pts_out, int dims)
{
    __shared__ int running[256];                       // next free output slot per digit
    __shared__ int wave_cnt[RS_WAVES][256];
    int lane = pccnn_lane();
    int wave = threadIdx.x >> 6;
    // first output slot of digit d for this tile = (keys with a smaller digit) + (same digit in earlier tiles)
    {
        const int tot = digit_totals[threadIdx.x];
        int incl = tot;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int t = __shfl_up(incl, o);
            if (lane >= o) incl += t;
        }
        if (lane == 63) wave_cnt[0][wave] = incl;
        __syncthreads();
        int add = 0;
#pragma unroll
        for (int w = 0; w < RS_WAVES; ++w)
            if (w < wave) add += wave_cnt[0][w];
        running[threadIdx.x] = add + incl - tot + tile_offsets[(int64_t)threadIdx.x * num_tiles + blockIdx.x];
        __syncthreads();
    }
#pragma unroll
    for (int w = 0; w < RS_WAVES; ++w) wave_cnt[w][threadIdx.x] = 0;
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * RS_THREADS * items;
    unsigned long long lt = pccnn_lanemask_lt();
    for (int r = 0; r < items; ++r) {
        int64_t i = base + r * RS_THREADS + threadIdx.x;
        bool valid = i < n;
        long long key = valid ? keys_in[i] : 0;
        int val = FIRST ? (int)i : (valid ? vals_in[i] : 0);
        int digit = (int)((key >> shift) & 0xff);
        // lanes of this wave holding the same digit
        unsigned long long peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            unsigned long long bal = __ballot((digit >> b) & 1);
            peers &= ((digit >> b) & 1) ? bal : ~bal;
        }
        int rank_in_wave = __popcll(peers & lt);
        if (valid && rank_in_wave == 0) wave_cnt[wave][digit] = __popcll(peers);
        __syncthreads();
        if (valid) {
            int dst = running[digit] + rank_in_wave;
#pragma unroll
            for (int w = 0; w < RS_WAVES; ++w)
                if (w < wave) dst += wave_cnt[w][digit];
            keys_out[dst] = key;
            vals_out[dst] = val;
            if (GATHER) {
#pragma unroll
                for (int k = 0; k < PCCNN_MAX_DIMS; ++k)
                    if (k < dims) pts_out[(int64_t)dst * dims + k] = pts[(int64_t)val * dims + k];
            }
        }
        __syncthreads();
        int tot = 0;
#pragma unroll
        for (int w = 0; w < RS_WAVES; ++w) {
            tot += wave_cnt[w][threadIdx.x];
            wave_cnt[w][threadIdx.x] = 0;
        }
        running[threadIdx.x] += tot;
        __syncthreads();
    }
}

extern "C" size_t pccnn_sort_keys_workspace_bytes(int64_t n)
{
    if (n < 0) n = 0;
    int64_t tiles = pccnn_ceil_div(n > 0 ? n : 1, (int64_t)RS_THREADS * rs_items_for(n));
    return pccnn_align((size_t)n * sizeof(int64_t)) + pccnn_align((size_t)n * sizeof(int32_t)) +
           pccnn_align((size_t)tiles * 256 * sizeof(int32_t)) + pccnn_align(256 * sizeof(int32_t)) + 256;
}

extern "C" int pccnn_sort_keys(const int64_t *keys, int64_t n, int key_bits, int64_t *sorted_keys_out,
                               int32_t *perm_out, const float *pts, int d, float *sorted_pts_out,
                               void *workspace, size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31), PCCNN_ERR_INVALID, "pccnn_sort_keys: n=%lld", (long long)n);
    PCCNN_REQUIRE((pts == nullptr) == (sorted_pts_out == nullptr), PCCNN_ERR_INVALID,
                  "pccnn_sort_keys: pts and sorted_pts_out must be given together");
    PCCNN_REQUIRE(pts == nullptr || (d >= 2 && d <= PCCNN_MAX_DIMS), PCCNN_ERR_UNSUPPORTED,
                  "pccnn_sort_keys: d=%d is not supported (2 <= d <= 6)", d);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(keys && sorted_keys_out && perm_out, PCCNN_ERR_INVALID, "pccnn_sort_keys: null pointer");
    PCCNN_REQUIRE(workspace_bytes >= pccnn_sort_keys_workspace_bytes(n), PCCNN_ERR_WORKSPACE,
                  "pccnn_sort_keys: workspace of %zu bytes, need %zu", workspace_bytes,
                  pccnn_sort_keys_workspace_bytes(n));
    hipStream_t s = (hipStream_t)stream;
    if (key_bits <= 0 || key_bits > 63) key_bits = 63;     // keys are non-negative
    int passes = (key_bits + 7) / 8;
    const int items = rs_items_for(n);
    int64_t tiles = pccnn_ceil_div(n, (int64_t)RS_THREADS * items);
    PccnnArena arena(workspace, workspace_bytes);
    int64_t *tmp_keys = arena.take<int64_t>((size_t)n);
    int32_t *tmp_vals = arena.take<int32_t>((size_t)n);
    int32_t *hist = arena.take<int32_t>((size_t)tiles * 256);
    int32_t *totals = arena.take<int32_t>(256);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_sort_keys: workspace too small");

    PccnnTimed timed(PCCNN_T_SORT, s);
    const int64_t *src_k = keys;
    const int32_t *src_v = nullptr;
    for (int p = 0; p < passes; ++p) {
        bool to_out = ((passes - 1 - p) % 2) == 0;
        int64_t *dst_k = to_out ? sorted_keys_out : tmp_keys;
        int32_t *dst_v = to_out ? perm_out : tmp_vals;
        int shift = 8 * p;
        bool last = (p == passes - 1);
        radix_hist_kernel<<<(unsigned)tiles, RS_THREADS, 0, s>>>(src_k, n, shift, items, hist, tiles);
        PCCNN_LAUNCH_CHECK();
        radix_scan_kernel<<<256, 256, 0, s>>>(hist, tiles, totals);
        PCCNN_LAUNCH_CHECK();
        bool gather = last && pts != nullptr;
        if (p == 0) {
            if (gather)
                radix_scatter_kernel<true, true><<<(unsigned)tiles, RS_THREADS, 0, s>>>(
                    src_k, src_v, n, shift, items, hist, tiles, totals, dst_k, dst_v, pts, sorted_pts_out, d);
            else
                radix_scatter_kernel<true, false><<<(unsigned)tiles, RS_THREADS, 0, s>>>(
                    src_k, src_v, n, shift, items, hist, tiles, totals, dst_k, dst_v, nullptr, nullptr, d);
        } else {
            if (gather)
                radix_scatter_kernel<false, true><<<(unsigned)tiles, RS_THREADS, 0, s>>>(
                    src_k, src_v, n, shift, items, hist, tiles, totals, dst_k, dst_v, pts, sorted_pts_out, d);
            else
                radix_scatter_kernel<false, false><<<(unsigned)tiles, RS_THREADS, 0, s>>>(
                    src_k, src_v, n, shift, items, hist, tiles, totals, dst_k, dst_v, nullptr, nullptr, d);
        }
        PCCNN_LAUNCH_CHECK();
        src_k = dst_k;
        src_v = dst_v;
    }
    return PCCNN_OK;
}
