// Stable LSD radix sort of (64-bit cell key, 32-bit index) pairs over the significant key bits only, 8 to 11
// bits per pass (see rs_plan).  Per pass:
//   1. radix_hist_kernel    : per-tile digit histogram staged in LDS, stored digit-major
//   2. radix_scan_kernel    : one workgroup per digit scans that digit's per-tile counts
//   3. radix_scatter_kernel : every tile re-reads its keys, ranks them with wave ballots
//                             (match-any on the digit bits), and scatters keys and indices;
//                             the last pass also gathers the xyz row of every point.
// Ties keep their input order in every pass, so the permutation is the stable argsort.
#include "common.h"

#define RS_THREADS 256
#define RS_MAX_ITEMS 8                                  // keys per thread and tile, at most
#define RS_STAGED_ITEMS RS_MAX_ITEMS                    // register arrays of the staged scatter kernel
#define RS_STAGED_FROM_ITEMS 3                          // tiles of this many keys per thread or more take the staged kernel
#define RS_WAVES (RS_THREADS / PCCNN_WAVE)

// Keys per thread of a tile: small inputs get small tiles, so that the launch still has a few hundred
// workgroups (a tile is walked in `items` rounds with barriers in between: few large tiles leave the chip
// idle), large inputs get the largest tiles (every tile pays a fixed set-up and a row of the histogram table).
static int rs_items_for(int64_t n)
{
    int64_t items = pccnn_ceil_div(n, (int64_t)RS_THREADS * 512);
    return (int)(items < 1 ? 1 : (items > RS_MAX_ITEMS ? RS_MAX_ITEMS : items));
}

// BITS bits per pass, D = 2^BITS digits; thread t of a workgroup looks after digits t, t + 256, ...
template <int BITS>
__global__ void __launch_bounds__(RS_THREADS)
radix_hist_kernel(const int64_t *__restrict__ keys, int64_t n, int shift, int items, int32_t *__restrict__ tile_hist,
                  int64_t num_tiles)
{
    constexpr int D = 1 << BITS;
    __shared__ int hist[D];
#pragma unroll
    for (int q = 0; q < D / RS_THREADS; ++q) hist[threadIdx.x + q * RS_THREADS] = 0;
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * RS_THREADS * items;
    for (int r = 0; r < items; ++r) {
        int64_t i = base + r * RS_THREADS + threadIdx.x;
        if (i < n) atomicAdd(&hist[(int)((keys[i] >> shift) & (D - 1))], 1);
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < D / RS_THREADS; ++q) {
        const int d = threadIdx.x + q * RS_THREADS;
        tile_hist[(int64_t)d * num_tiles + blockIdx.x] = hist[d];
    }
}

// The first pass's histogram for keys that do not exist yet: the tile computes the cell keys of its points (the
// arithmetic of compute_keys_kernel), stores them for the scatter that follows, and counts their lowest digit.
template <int BITS>
__global__ void __launch_bounds__(RS_THREADS)
radix_hist_keys_kernel(PccnnKeySource src, int64_t *__restrict__ keys, int64_t n, int items,
                       int32_t *__restrict__ tile_hist, int64_t num_tiles)
{
    constexpr int D = 1 << BITS;
    __shared__ int hist[D];
#pragma unroll
    for (int q = 0; q < D / RS_THREADS; ++q) hist[threadIdx.x + q * RS_THREADS] = 0;
    int nc[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) nc[k] = src.use_sized ? src.sized.v[k] : src.num_cells[k];
    if (src.use_sized && blockIdx.x == 0 && threadIdx.x < 3) src.num_cells_out[threadIdx.x] = src.sized.v[threadIdx.x];
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * RS_THREADS * items;
    for (int r = 0; r < items; ++r) {
        int64_t i = base + r * RS_THREADS + threadIdx.x;
        if (i < n) {
            const long long key = pccnn_point_key3(src.pts, src.batch_ids, src.aabb_min, src.cell_size, nc, i);
            keys[i] = key;
            atomicAdd(&hist[(int)(key & (D - 1))], 1);
        }
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < D / RS_THREADS; ++q) {
        const int d = threadIdx.x + q * RS_THREADS;
        tile_hist[(int64_t)d * num_tiles + blockIdx.x] = hist[d];
    }
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
        const int incl = pccnn_wave_inclusive_scan_i(x);
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

template <int BITS, bool FIRST, bool GATHER>
__global__ void __launch_bounds__(RS_THREADS)
radix_scatter_kernel(const int64_t *__restrict__ keys_in, const int32_t *__restrict__ vals_in, int64_t n, int shift,
                     int items, const int32_t *__restrict__ tile_offsets, int64_t num_tiles,
                     const int32_t *__restrict__ digit_totals, int64_t *__restrict__ keys_out, int32_t *__restrict__ vals_out,
                     const float *__restrict__ pts, float *__restrict__ pts_out, int dims)
{
    constexpr int D = 1 << BITS;
    constexpr int PER = D / RS_THREADS;
    __shared__ int running[D];                         // next free output slot per digit
    __shared__ int wave_cnt[RS_WAVES][D];
    int lane = pccnn_lane();
    int wave = threadIdx.x >> 6;
    // first output slot of digit d for this tile = (keys with a smaller digit) + (same digit in earlier tiles);
    // for this prefix thread t takes the PER consecutive digits t * PER ...
    // digit_totals == nullptr (few tiles): tile_offsets is the histogram pass's table as it stands, and every
    // workgroup adds up its digits' rows itself - the row's total and the part before its own tile - instead of a
    // scan launch in between.
    {
        int tot[PER], before[PER];
        int sum = 0;
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int d = threadIdx.x * PER + q;
            if (digit_totals != nullptr) {
                tot[q] = digit_totals[d];
                before[q] = tile_offsets[(int64_t)d * num_tiles + blockIdx.x];
            } else {
                int all = 0, mine = 0;
                for (int64_t t = 0; t < num_tiles; ++t) {
                    const int v = tile_offsets[(int64_t)d * num_tiles + t];
                    all += v;
                    if (t < (int64_t)blockIdx.x) mine += v;
                }
                tot[q] = all;
                before[q] = mine;
            }
            sum += tot[q];
        }
        const int incl = pccnn_wave_inclusive_scan_i(sum);
        if (lane == 63) wave_cnt[0][wave] = incl;
        __syncthreads();
        int excl = incl - sum;
#pragma unroll
        for (int w = 0; w < RS_WAVES; ++w)
            if (w < wave) excl += wave_cnt[0][w];
        __syncthreads();
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int d = threadIdx.x * PER + q;
            running[d] = excl + before[q];
            excl += tot[q];
        }
    }
#pragma unroll
    for (int w = 0; w < RS_WAVES; ++w)
#pragma unroll
        for (int q = 0; q < PER; ++q) wave_cnt[w][threadIdx.x + q * RS_THREADS] = 0;
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * RS_THREADS * items;
    unsigned long long lt = pccnn_lanemask_lt();
    for (int r = 0; r < items; ++r) {
        int64_t i = base + r * RS_THREADS + threadIdx.x;
        bool valid = i < n;
        long long key = valid ? keys_in[i] : 0;
        int val = FIRST ? (int)i : (valid ? vals_in[i] : 0);
        int digit = (int)((key >> shift) & (D - 1));
        // lanes of this wave holding the same digit
        unsigned long long peers = __ballot(valid);
#pragma unroll
        for (int b = 0; b < BITS; ++b) {
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
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            const int d = threadIdx.x + q * RS_THREADS;
            int tot = 0;
#pragma unroll
            for (int w = 0; w < RS_WAVES; ++w) {
                tot += wave_cnt[w][d];
                wave_cnt[w][d] = 0;
            }
            running[d] += tot;
        }
        __syncthreads();
    }
}

// The scatter pass for large inputs.  Same job as radix_scatter_kernel (the slot of every key = keys with a smaller
// digit + keys of the same digit in earlier tiles + its rank among the tile's keys of that digit), laid out
// differently:
//  * a wavefront owns items * 64 consecutive keys and ranks them against its own LDS counters, round after round
//    without a workgroup barrier (a wavefront's LDS accesses execute in order); one barrier and one prefix over the
//    waves then turn the counters into places inside the tile;
//  * the tile is parked in LDS in sorted order and written out from there: the keys of one digit are consecutive
//    in the tile and consecutive at their destination, so a run leaves as consecutive addresses from consecutive
//    lanes instead of one 8-byte and one 4-byte store per lane wherever its key happens to go.
template <int BITS, bool FIRST, bool GATHER>
__global__ void __launch_bounds__(RS_THREADS)
radix_scatter_staged_kernel(const int64_t *__restrict__ keys_in, const int32_t *__restrict__ vals_in, int64_t n, int shift,
                            int items, const int32_t *__restrict__ tile_offsets, int64_t num_tiles,
                            const int32_t *__restrict__ digit_totals, int64_t *__restrict__ keys_out,
                            int32_t *__restrict__ vals_out, const float *__restrict__ pts, float *__restrict__ pts_out,
                            int dims)
{
    constexpr int D = 1 << BITS;
    constexpr int PER = D / RS_THREADS;                // digits per thread: tid * PER ... tid * PER + PER - 1
    constexpr int STAGE_BYTES = RS_THREADS * RS_STAGED_ITEMS * 12;
    constexpr int CNT_BYTES = RS_WAVES * D * 4;
    __shared__ __align__(16) unsigned char lds[(STAGE_BYTES > CNT_BYTES ? STAGE_BYTES : CNT_BYTES) + D * 4 + 64];
    volatile int *cnt = (volatile int *)lds;                                       // [RS_WAVES][D]; later the staging area
    const int tile_keys = RS_THREADS * items;
    long long *stage_keys = (long long *)lds;                                     // [tile_keys]
    int *stage_vals = (int *)(lds + (size_t)tile_keys * 8);                       // [tile_keys]
    int *base = (int *)(lds + (STAGE_BYTES > CNT_BYTES ? STAGE_BYTES : CNT_BYTES)); // [D] slot of the tile's j-th key = base[digit] + j
    int *misc = base + D;                                                         // [16]

    const int tid = threadIdx.x, lane = pccnn_lane(), wave = tid >> 6;
    const int64_t tile = blockIdx.x;
    for (int i = tid; i < RS_WAVES * D; i += RS_THREADS) cnt[i] = 0;
    const int64_t tile_base = tile * tile_keys;
    const int64_t wave_base = tile_base + (int64_t)wave * items * 64;
    long long key[RS_STAGED_ITEMS];
    int val[RS_STAGED_ITEMS], rnk[RS_STAGED_ITEMS];
#pragma unroll
    for (int r = 0; r < RS_STAGED_ITEMS; ++r) {
        key[r] = 0;
        val[r] = -1;                                                  // -1 = no key in this slot
        if (r < items) {
            const int64_t i = wave_base + r * 64 + lane;
            if (i < n) {
                key[r] = keys_in[i];
                val[r] = FIRST ? (int)i : vals_in[i];
            }
        }
    }
    __syncthreads();                                                  // counters are zero
    const unsigned long long lt = pccnn_lanemask_lt();
#pragma unroll
    for (int r = 0; r < RS_STAGED_ITEMS; ++r) {
        rnk[r] = 0;
        if (r < items) {
            const bool valid = val[r] >= 0;
            const int digit = (int)((key[r] >> shift) & (D - 1));
            unsigned long long peers = __ballot(valid);               // lanes of this wave holding the same digit
#pragma unroll
            for (int b = 0; b < BITS; ++b) {
                const unsigned long long bal = __ballot((digit >> b) & 1);
                peers &= ((digit >> b) & 1) ? bal : ~bal;
            }
            const int rank_in_wave = __popcll(peers & lt);
            // every lane reads the counter before the first of its peers moves it on
            const int before = valid ? cnt[wave * D + digit] : 0;
            __builtin_amdgcn_wave_barrier();
            if (valid && rank_in_wave == 0) cnt[wave * D + digit] = before + __popcll(peers);
            __builtin_amdgcn_wave_barrier();
            rnk[r] = before + rank_in_wave;
        }
    }
    __syncthreads();
    // per digit: the tile's count and the waves' shares of it; prefix over the digits of both the tile's counts
    // and the totals of all tiles
    int tot[PER], glob[PER], wcnt[PER][RS_WAVES];
    int sum_tot = 0, sum_glob = 0;
#pragma unroll
    for (int q = 0; q < PER; ++q) {
        const int d = tid * PER + q;
        tot[q] = 0;
#pragma unroll
        for (int w = 0; w < RS_WAVES; ++w) {
            wcnt[q][w] = cnt[w * D + d];
            tot[q] += wcnt[q][w];
        }
        glob[q] = digit_totals[d];
        sum_tot += tot[q];
        sum_glob += glob[q];
    }
    int local_start = sum_tot, global_start = sum_glob;
    {
        const int ia = pccnn_wave_inclusive_scan_i(local_start), ib = pccnn_wave_inclusive_scan_i(global_start);
        if (lane == 63) { misc[wave] = ia; misc[RS_WAVES + wave] = ib; }
        __syncthreads();
        int pa = 0, pb = 0;
#pragma unroll
        for (int w = 0; w < RS_WAVES; ++w)
            if (w < wave) { pa += misc[w]; pb += misc[RS_WAVES + w]; }
        local_start = pa + ia - local_start;                          // exclusive, of this thread's first digit
        global_start = pb + ib - global_start;
    }
#pragma unroll
    for (int q = 0; q < PER; ++q) {
        const int d = tid * PER + q;
        base[d] = global_start + tile_offsets[(int64_t)d * num_tiles + tile] - local_start;
        int at = local_start;
#pragma unroll
        for (int w = 0; w < RS_WAVES; ++w) {
            cnt[w * D + d] = at;                                      // place of wave w's first key with digit d
            at += wcnt[q][w];
        }
        local_start += tot[q];
        global_start += glob[q];
    }
    __syncthreads();
    int pos[RS_STAGED_ITEMS];
#pragma unroll
    for (int r = 0; r < RS_STAGED_ITEMS; ++r) {
        pos[r] = 0;
        if (r < items && val[r] >= 0) pos[r] = cnt[wave * D + (int)((key[r] >> shift) & (D - 1))] + rnk[r];
    }
    __syncthreads();                                                  // cnt is dead: its memory becomes the staging area
#pragma unroll
    for (int r = 0; r < RS_STAGED_ITEMS; ++r) {
        if (r < items && val[r] >= 0) {
            stage_keys[pos[r]] = key[r];
            stage_vals[pos[r]] = val[r];
        }
    }
    __syncthreads();
    const int64_t left = n - tile_base;
    const int tile_count = left < tile_keys ? (int)left : tile_keys;
    for (int j = tid; j < tile_count; j += RS_THREADS) {
        const long long k = stage_keys[j];
        const int v = stage_vals[j];
        const int64_t dst = (int64_t)base[(int)((k >> shift) & (D - 1))] + j;
        keys_out[dst] = k;
        vals_out[dst] = v;
        if (GATHER) {
#pragma unroll
            for (int c = 0; c < PCCNN_MAX_DIMS; ++c)
                if (c < dims) pts_out[dst * dims + c] = pts[(int64_t)v * dims + c];
        }
    }
}

// Passes and bits per pass for keys of `key_bits` significant bits: as few passes as the widest digit allows,
// the bits spread evenly over them (18 bits: 2 x 9; 24: 3 x 8).  Wide digits pay where a pass is bound by its three
// launches: up to 11 bits for at most 2^18 keys (65 536 keys of 18 bits: 26 us in 2 passes against 35 us in 3).
// On a million keys a pass with 2^11 digits leaves two keys per digit and tile, its scattered stores and the
// larger table cost more than the saved pass (22 bits: 116 us in 2 passes against 99 us in 3), and 9 bits are the
// widest digit that still wins (800 000 keys of 18 bits: 72 us against 80 us).
#define RS_SELF_SCAN_TILES 64           // tiles up to which the scatter does the scan's job itself
#define RS_MAX_BITS 11
#define RS_MAX_DIGITS (1 << RS_MAX_BITS)
static void rs_plan(int key_bits, int64_t n, int &passes, int &bits)
{
    const int widest = n <= (1 << 18) ? RS_MAX_BITS : 9;
    passes = (key_bits + widest - 1) / widest;
    bits = (key_bits + passes - 1) / passes;
    if (bits < 8) bits = 8;
}

extern "C" size_t pccnn_sort_keys_workspace_bytes(int64_t n)
{
    if (n < 0) n = 0;
    int64_t tiles = pccnn_ceil_div(n > 0 ? n : 1, (int64_t)RS_THREADS * rs_items_for(n));
    return pccnn_align((size_t)n * sizeof(int64_t)) + pccnn_align((size_t)n * sizeof(int32_t)) +
           pccnn_align((size_t)tiles * RS_MAX_DIGITS * sizeof(int32_t)) + pccnn_align(RS_MAX_DIGITS * sizeof(int32_t)) + 256;
}

// The sort proper; `timed` = bracket the launches with the optional timing events (which are created on the fly,
// so the entry point that must not allocate anything passes false).
// `make_keys` (nullable): the keys do not exist yet; the first histogram pass computes them into `keys`.
static int sort_keys_run(const int64_t *keys, int64_t n, int key_bits, int64_t *sorted_keys_out, int32_t *perm_out,
                         const float *pts, int d, float *sorted_pts_out, void *workspace, size_t workspace_bytes,
                         void *stream, bool timed_on, const PccnnKeySource *make_keys = nullptr)
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
    int passes, bits;
    rs_plan(key_bits, n, passes, bits);
    const int items = rs_items_for(n);
    int64_t tiles = pccnn_ceil_div(n, (int64_t)RS_THREADS * items);
    PccnnArena arena(workspace, workspace_bytes);
    int64_t *tmp_keys = arena.take<int64_t>((size_t)n);
    int32_t *tmp_vals = arena.take<int32_t>((size_t)n);
    int32_t *hist = arena.take<int32_t>((size_t)tiles * RS_MAX_DIGITS);
    int32_t *totals = arena.take<int32_t>(RS_MAX_DIGITS);
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_sort_keys: workspace too small");

    PccnnTimed timed(timed_on ? PCCNN_T_SORT : -1, s);
    // measured: the staged scatter wins from about 300 000 keys on (84 against 99 us at 10^6 keys of 22 bits),
    // the plain one below that (27 against 30 us at 65 536 keys), where a tile's fixed work outweighs its stores
    const bool staged = items >= RS_STAGED_FROM_ITEMS;
    // few tiles: the scatter's workgroups add up the histogram rows themselves, no scan launch
    const bool self_scan = !staged && tiles <= RS_SELF_SCAN_TILES;
    const int64_t *src_k = keys;
    const int32_t *src_v = nullptr;
    for (int p = 0; p < passes; ++p) {
        bool to_out = ((passes - 1 - p) % 2) == 0;
        int64_t *dst_k = to_out ? sorted_keys_out : tmp_keys;
        int32_t *dst_v = to_out ? perm_out : tmp_vals;
        int shift = bits * p;
        bool last = (p == passes - 1);
        bool gather = last && pts != nullptr;
        const unsigned grid = (unsigned)tiles;
#define RS_SCATTER(B, FIRST, GATHER)                                                                            \
    do {                                                                                                          \
        if (staged)                                                                                               \
            radix_scatter_staged_kernel<B, FIRST, GATHER><<<grid, RS_THREADS, 0, s>>>(                            \
                src_k, src_v, n, shift, items, hist, tiles, totals, dst_k, dst_v, GATHER ? pts : nullptr,         \
                GATHER ? sorted_pts_out : nullptr, d);                                                            \
        else                                                                                                      \
            radix_scatter_kernel<B, FIRST, GATHER><<<grid, RS_THREADS, 0, s>>>(                                   \
                src_k, src_v, n, shift, items, hist, tiles, self_scan ? nullptr : totals, dst_k, dst_v,           \
                GATHER ? pts : nullptr, GATHER ? sorted_pts_out : nullptr, d);                                    \
    } while (0)
#define RS_PASS(B)                                                                                   \
    do {                                                                                             \
        if (p == 0 && make_keys != nullptr)                                                          \
            radix_hist_keys_kernel<B><<<grid, RS_THREADS, 0, s>>>(*make_keys, (int64_t *)keys, n, items, hist, tiles); \
        else                                                                                         \
            radix_hist_kernel<B><<<grid, RS_THREADS, 0, s>>>(src_k, n, shift, items, hist, tiles);   \
        PCCNN_LAUNCH_CHECK();                                                                        \
        if (!self_scan) radix_scan_kernel<<<1 << B, 256, 0, s>>>(hist, tiles, totals);               \
        PCCNN_LAUNCH_CHECK();                                                                        \
        if (p == 0) {                                                                                \
            if (gather) RS_SCATTER(B, true, true); else RS_SCATTER(B, true, false);                  \
        } else {                                                                                     \
            if (gather) RS_SCATTER(B, false, true); else RS_SCATTER(B, false, false);                \
        }                                                                                            \
        PCCNN_LAUNCH_CHECK();                                                                        \
    } while (0)
        switch (bits) {
        case 8: RS_PASS(8); break;
        case 9: RS_PASS(9); break;
        case 10: RS_PASS(10); break;
        default: RS_PASS(11); break;
        }
#undef RS_PASS
#undef RS_SCATTER
        src_k = dst_k;
        src_v = dst_v;
    }
    return PCCNN_OK;
}

extern "C" int pccnn_sort_keys(const int64_t *keys, int64_t n, int key_bits, int64_t *sorted_keys_out,
                               int32_t *perm_out, const float *pts, int d, float *sorted_pts_out,
                               void *workspace, size_t workspace_bytes, void *stream)
{
    return sort_keys_run(keys, n, key_bits, sorted_keys_out, perm_out, pts, d, sorted_pts_out, workspace,
                         workspace_bytes, stream, true);
}

int pccnn_sort_keys_from_points(const PccnnKeySource &source, int64_t *keys_out, int64_t n, int key_bits,
                                int64_t *sorted_keys_out, int32_t *perm_out, float *sorted_pts_out, void *workspace,
                                size_t workspace_bytes, void *stream)
{
    PCCNN_REQUIRE(source.pts && source.batch_ids && source.aabb_min && source.cell_size &&
                      (source.use_sized ? source.num_cells_out != nullptr : source.num_cells != nullptr),
                  PCCNN_ERR_INVALID, "pccnn_grid_build: null pointer");
    return sort_keys_run(keys_out, n, key_bits, sorted_keys_out, perm_out, source.pts, 3, sorted_pts_out, workspace,
                         workspace_bytes, stream, true, &source);
}

// ---- the same sort for callers that cannot allocate device memory ---------------------------------------------
// Its workspace is a fixed array in the library's device image, one copy per GPU, held until the process ends.
// In host code the array's name is only a handle: the device address of the current GPU's copy comes from
// hipGetSymbolAddress, once per device, and that pointer is what the kernels, fills and copies get.
#include <mutex>

#define SORT_SCRATCH_BYTES                                                                                          \
    ((size_t)PCCNN_SORT_KEYS_STATIC_MAX * 8 + (size_t)PCCNN_SORT_KEYS_STATIC_MAX * 4 +                              \
     (size_t)(PCCNN_SORT_KEYS_STATIC_MAX / (RS_THREADS * RS_MAX_ITEMS)) * RS_MAX_DIGITS * 4 + RS_MAX_DIGITS * 4 + 1024)
static __device__ __align__(256) unsigned char scratch[SORT_SCRATCH_BYTES];

#define SORT_MAX_DEVICES 64
static std::mutex g_scratch_mu;
static void *g_scratch_ptr[SORT_MAX_DEVICES];          // device address of `scratch` on each GPU, 0 = not asked yet

static int scratch_of_current_device(void **out)
{
    int dev = -1;
    PCCNN_HIP_CHECK(hipGetDevice(&dev));
    PCCNN_REQUIRE(dev >= 0 && dev < SORT_MAX_DEVICES, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_sort_keys_static: device %d is beyond the %d devices this build keeps a scratch pointer for",
                  dev, SORT_MAX_DEVICES);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *p = nullptr;
        PCCNN_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        PCCNN_REQUIRE(p != nullptr, PCCNN_ERR_HIP, "pccnn_sort_keys_static: the scratch array has no device address");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return PCCNN_OK;
}

extern "C" int pccnn_sort_keys_static(const int64_t *keys, int64_t n, int key_bits, int64_t *sorted_keys_out,
                                      int32_t *perm_out, const float *pts, int d, float *sorted_pts_out, void *stream)
{
    PCCNN_REQUIRE(n >= 0 && n <= PCCNN_SORT_KEYS_STATIC_MAX, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_sort_keys_static: n=%lld keys, the built-in scratch holds at most %d; use pccnn_sort_keys with "
                  "a workspace for more", (long long)n, PCCNN_SORT_KEYS_STATIC_MAX);
    PCCNN_REQUIRE(pccnn_sort_keys_workspace_bytes(n) <= SORT_SCRATCH_BYTES, PCCNN_ERR_UNSUPPORTED,
                  "pccnn_sort_keys_static: %zu bytes of scratch needed, %zu built in",
                  pccnn_sort_keys_workspace_bytes(n), (size_t)SORT_SCRATCH_BYTES);
    void *ws = nullptr;
    int rc = scratch_of_current_device(&ws);
    if (rc != PCCNN_OK) return rc;
    // every piece of the scratch that a pass reads is written by that pass first: nothing has to start at zero
    return sort_keys_run(keys, n, key_bits, sorted_keys_out, perm_out, pts, d, sorted_pts_out, ws, SORT_SCRATCH_BYTES,
                         stream, false);
}
