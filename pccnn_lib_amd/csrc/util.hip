// Error reporting, fill kernels and the device-wide int32 scan shared by the other files.
#include <stdarg.h>

#include "common.h"

static thread_local char g_err[512] = "";

void pccnn_set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char *pccnn_last_error(void) { return g_err; }
extern "C" int pccnn_version(void) { return 1; }

// ----------------------------------------------------------------- timing

#include <mutex>
#include <vector>

static bool g_timing_on = false;
static std::mutex g_timing_mu;
struct TimedPair { hipEvent_t start, stop; };
static std::vector<TimedPair> g_timing_pending[PCCNN_T_COUNT];
static double g_timing_ms[PCCNN_T_COUNT];
static long long g_timing_n[PCCNN_T_COUNT];
static const char *g_timing_names[PCCNN_T_COUNT] = {"gemm", "proj_fwd", "proj_bwd", "basis_bwd", "nb_count",
                                                    "nb_fill",  "sort",     "keys",     "grid",      "pdf", "scan",
                                                    "fused_fwd"};

PccnnTimed::PccnnTimed(int id_, hipStream_t s) : id(id_), stream(s), stop(nullptr), on(g_timing_on && id_ >= 0)
{
    if (!on) return;
    hipEvent_t start;
    if (hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess) { on = false; return; }
    (void)hipEventRecord(start, stream);
    std::lock_guard<std::mutex> lk(g_timing_mu);
    g_timing_pending[id].push_back({start, stop});
}

PccnnTimed::~PccnnTimed()
{
    if (on) (void)hipEventRecord(stop, stream);
}

static void timing_drain()
{
    for (int i = 0; i < PCCNN_T_COUNT; ++i) {
        for (auto &pr : g_timing_pending[i]) {
            float ms = 0.0f;
            if (hipEventSynchronize(pr.stop) == hipSuccess && hipEventElapsedTime(&ms, pr.start, pr.stop) == hipSuccess) {
                g_timing_ms[i] += ms;
                g_timing_n[i] += 1;
            }
            (void)hipEventDestroy(pr.start);
            (void)hipEventDestroy(pr.stop);
        }
        g_timing_pending[i].clear();
    }
}

extern "C" int pccnn_timing_enable(int on)
{
    std::lock_guard<std::mutex> lk(g_timing_mu);
    timing_drain();
    g_timing_on = on != 0;
    return PCCNN_OK;
}

extern "C" int pccnn_timing_reset(void)
{
    std::lock_guard<std::mutex> lk(g_timing_mu);
    timing_drain();
    for (int i = 0; i < PCCNN_T_COUNT; ++i) { g_timing_ms[i] = 0.0; g_timing_n[i] = 0; }
    return PCCNN_OK;
}

extern "C" int pccnn_timing_count(void) { return PCCNN_T_COUNT; }

extern "C" const char *pccnn_timing_name(int id) { return (id >= 0 && id < PCCNN_T_COUNT) ? g_timing_names[id] : ""; }

extern "C" int pccnn_timing_read(int id, int64_t *h_launches, double *h_total_ms)
{
    PCCNN_REQUIRE(id >= 0 && id < PCCNN_T_COUNT && h_launches && h_total_ms, PCCNN_ERR_INVALID,
                  "pccnn_timing_read: bad timer id %d or null output", id);
    std::lock_guard<std::mutex> lk(g_timing_mu);
    timing_drain();
    *h_launches = g_timing_n[id];
    *h_total_ms = g_timing_ms[id];
    return PCCNN_OK;
}

// ------------------------------------------------------------------ fills

template <typename T> __global__ void fill_kernel(T *p, T v, int64_t n)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}

template <typename T> static int fill_impl(T *p, T v, int64_t n, hipStream_t s)
{
    if (n <= 0) return PCCNN_OK;
    int64_t blocks = pccnn_ceil_div(n, 256);
    if (blocks > 8192) blocks = 8192;
    fill_kernel<T><<<(unsigned)blocks, 256, 0, s>>>(p, v, n);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

int pccnn_fill_i32(int32_t *p, int32_t v, int64_t n, hipStream_t s) { return fill_impl<int32_t>(p, v, n, s); }
int pccnn_fill_f32(float *p, float v, int64_t n, hipStream_t s) { return fill_impl<float>(p, v, n, s); }

// A plain float4 copy: the known-size yardstick that hardware traffic counters are scaled against.
__global__ void __launch_bounds__(256) calibration_copy_kernel(const float4 *__restrict__ src,
                                                               float4 *__restrict__ dst, int64_t n4)
{
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += stride) dst[i] = src[i];
}

extern "C" int pccnn_calibration_copy(const float *src, float *dst, int64_t count, void *stream)
{
    PCCNN_REQUIRE(count >= 0 && count % 4 == 0, PCCNN_ERR_INVALID, "pccnn_calibration_copy: count=%lld must be a multiple of 4",
                  (long long)count);
    if (count == 0) return PCCNN_OK;
    PCCNN_REQUIRE(src && dst && (uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0, PCCNN_ERR_INVALID,
                  "pccnn_calibration_copy: null or unaligned pointer");
    int64_t blocks = pccnn_ceil_div(count / 4, 256);
    if (blocks > 16384) blocks = 16384;
    calibration_copy_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const float4 *)src, (float4 *)dst, count / 4);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// ------------------------------------------------------------------- row permutation
// dst[i, :] = src[index[i], :] for rows of `row_floats` floats: one lane per 16 bytes when the rows allow it.
template <typename V>
__global__ void __launch_bounds__(256)
gather_rows_kernel(const V *__restrict__ src, const int32_t *__restrict__ index, V *__restrict__ dst, int64_t rows,
                   int per_row, int64_t src_rows)
{
    const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= rows * per_row) return;
    const int64_t r = e / per_row;
    const int c = (int)(e % per_row);
    const int64_t from = index[r];
    if (from >= 0 && from < src_rows) dst[e] = src[from * per_row + c];
}

extern "C" int pccnn_gather_rows_f32(const float *src, const int32_t *index, float *dst, int64_t rows, int row_floats,
                                     int64_t src_rows, void *stream)
{
    PCCNN_REQUIRE(rows >= 0 && row_floats >= 1 && src_rows >= 0, PCCNN_ERR_INVALID,
                  "pccnn_gather_rows_f32: rows=%lld row_floats=%d src_rows=%lld", (long long)rows, row_floats,
                  (long long)src_rows);
    if (rows == 0) return PCCNN_OK;
    PCCNN_REQUIRE(src && index && dst, PCCNN_ERR_INVALID, "pccnn_gather_rows_f32: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const bool wide = row_floats % 4 == 0 && (uintptr_t)src % 16 == 0 && (uintptr_t)dst % 16 == 0;
    const int per_row = wide ? row_floats / 4 : row_floats;
    const int64_t blocks = pccnn_ceil_div(rows * per_row, 256);
    PCCNN_REQUIRE(blocks < (1ll << 31), PCCNN_ERR_UNSUPPORTED, "pccnn_gather_rows_f32: too many elements");
    if (wide)
        gather_rows_kernel<float4><<<(unsigned)blocks, 256, 0, s>>>((const float4 *)src, index, (float4 *)dst, rows,
                                                                   per_row, src_rows);
    else
        gather_rows_kernel<float><<<(unsigned)blocks, 256, 0, s>>>(src, index, dst, rows, per_row, src_rows);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// inverse[perm[i]] = i
__global__ void __launch_bounds__(256)
invert_permutation_kernel(const int32_t *__restrict__ perm, int32_t *__restrict__ inverse, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int64_t to = perm[i];
    if (to >= 0 && to < n) inverse[to] = (int32_t)i;
}

extern "C" int pccnn_invert_permutation_i32(const int32_t *perm, int32_t *inverse, int64_t n, void *stream)
{
    PCCNN_REQUIRE(n >= 0 && n < (1ll << 31), PCCNN_ERR_INVALID, "pccnn_invert_permutation_i32: n=%lld", (long long)n);
    if (n == 0) return PCCNN_OK;
    PCCNN_REQUIRE(perm && inverse, PCCNN_ERR_INVALID, "pccnn_invert_permutation_i32: null pointer");
    invert_permutation_kernel<<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(perm, inverse, n);
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}

// ------------------------------------------------------------------- scan
// Three launches: per-tile inclusive scan + tile totals, scan of the totals by one
// workgroup, add of the tile prefix.  Tiles are SCAN_TILE consecutive elements.

#define SCAN_THREADS 256
#define SCAN_ITEMS 8
#define SCAN_TILE (SCAN_THREADS * SCAN_ITEMS)

// int32 tile sums, then (8-byte aligned) the 64-bit sums of the same tiles
size_t pccnn_scan_tmp_elems(int64_t n) { return 3 * ((size_t)pccnn_ceil_div(n > 0 ? n : 1, SCAN_TILE) + 2); }

// Inclusive scan of one value per thread across a 256-thread workgroup.
__device__ __forceinline__ int block_inclusive_scan(int v, int *lds /* >= 4 ints */, int &total)
{
    int lane = pccnn_lane();
    int wave = threadIdx.x >> 6;
    v = pccnn_wave_inclusive_scan_i(v);
    if (lane == 63) lds[wave] = v;
    __syncthreads();
    int add = 0;
    int tot = 0;
#pragma unroll
    for (int w = 0; w < SCAN_THREADS / 64; ++w) {
        int x = lds[w];
        if (w < wave) add += x;
        tot += x;
    }
    total = tot;
    __syncthreads();
    return v + add;
}

// Sum of one 64-bit value per thread across the workgroup, returned in every thread of wavefront 0.
__device__ __forceinline__ long long block_sum_i64(long long v, long long *lds /* >= 4 */)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if (pccnn_lane() == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    long long tot = 0;
#pragma unroll
    for (int w = 0; w < SCAN_THREADS / 64; ++w) tot += lds[w];
    __syncthreads();
    return tot;
}

// tile_sums64 (nullable): the same tile totals without the 32-bit wrap-around, for the caller that has to know
// whether the running totals still fit 31 bits.
__global__ void __launch_bounds__(SCAN_THREADS)
scan_tiles_kernel(const int32_t *__restrict__ in, int32_t *__restrict__ out, int64_t n, int clamp_max,
                  int32_t *__restrict__ tile_sums, long long *__restrict__ tile_sums64)
{
    __shared__ int lds[4];
    __shared__ long long lds64[4];
    int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    int v[SCAN_ITEMS];
    int sum = 0;
    long long wide = 0;                 // the tile's sum in 64 bits, from the same loads (in may alias out)
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
        int x = (base + i < n) ? in[base + i] : 0;
        if (clamp_max > 0 && x > clamp_max) x = clamp_max;
        wide += x;
        sum += x;
        v[i] = sum;
    }
    int total;
    int incl = block_inclusive_scan(sum, lds, total);
    int excl = incl - sum;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i)
        if (base + i < n) out[base + i] = v[i] + excl;
    if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
    if (tile_sums64) {
        wide = block_sum_i64(wide, lds64);
        if (threadIdx.x == 0) tile_sums64[blockIdx.x] = wide;
    }
}

// Exclusive scan of the tile totals, in place, by a single workgroup.
// total_out (nullable): the sum of the 64-bit tile sums.
__global__ void __launch_bounds__(SCAN_THREADS)
scan_tile_sums_kernel(int32_t *__restrict__ tile_sums, int64_t num_tiles, const long long *__restrict__ tile_sums64,
                      long long *__restrict__ total_out)
{
    __shared__ int lds[4];
    __shared__ long long lds64[4];
    if (total_out) {
        long long v = 0;
        for (int64_t i = threadIdx.x; i < num_tiles; i += SCAN_THREADS) v += tile_sums64[i];
        v = block_sum_i64(v, lds64);
        if (threadIdx.x == 0) total_out[0] = v;
    }
    int carry = 0;
    for (int64_t base = 0; base < num_tiles; base += SCAN_THREADS) {
        int64_t i = base + threadIdx.x;
        int x = (i < num_tiles) ? tile_sums[i] : 0;
        int total;
        int incl = block_inclusive_scan(x, lds, total);
        if (i < num_tiles) tile_sums[i] = carry + incl - x;
        carry += total;
    }
}

__global__ void __launch_bounds__(SCAN_THREADS)
scan_add_kernel(int32_t *__restrict__ out, int64_t n, const int32_t *__restrict__ tile_sums)
{
    int add = tile_sums[blockIdx.x];
    int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i)
        if (base + i < n) out[base + i] += add;
}

// Up to SCAN_SMALL_MAX elements: one workgroup of 1024 threads, one launch instead of three (each of which runs for
// 4 to 6 us whatever its size).  Every wavefront owns ITEMS (4 to 48) consecutive rows of 64 elements and requests
// them all before it adds anything (lane = column: every load and store is one contiguous 256-byte row), scans row
// after row (pccnn_wave_inclusive_scan_i) with a running total, and the 16 wavefronts' totals meet in LDS: one memory round
// trip, ITEMS row scans, one exchange, the stores.
#define SCAN_SMALL_THREADS 1024
#define SCAN_SMALL_MAX (48 * SCAN_SMALL_THREADS)

template <int ITEMS>
__global__ void __launch_bounds__(SCAN_SMALL_THREADS)
scan_small_kernel(const int32_t *__restrict__ in, int32_t *__restrict__ out, int64_t n, int clamp_max,
                  long long *__restrict__ total_out)
{
    constexpr int WAVES = SCAN_SMALL_THREADS / 64;
    __shared__ int wave_sum[WAVES];
    __shared__ long long wave_wide[WAVES];
    const int lane = pccnn_lane(), wave = threadIdx.x >> 6;
    const int64_t base = (int64_t)wave * ITEMS * 64 + lane;
    int v[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) v[i] = (base + i * 64 < n) ? in[base + i * 64] : 0;
    int carry = 0;
    long long wide = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        int x = v[i];
        if (clamp_max > 0 && x > clamp_max) x = clamp_max;
        wide += x;
        x = pccnn_wave_inclusive_scan_i(x);
        v[i] = x + carry;
        carry += pccnn_bcast_i(x, 63);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) wide += __shfl_xor(wide, o);
    if (lane == 0) { wave_sum[wave] = carry; wave_wide[wave] = wide; }
    __syncthreads();
    int before = 0;
    long long total = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        if (w < wave) before += wave_sum[w];
        total += wave_wide[w];
    }
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
        if (base + i * 64 < n) out[base + i * 64] = v[i] + before;
    if (total_out && threadIdx.x == 0) total_out[0] = total;
}

int pccnn_scan_inclusive_i32(const int32_t *in, int32_t *out, int64_t n, int clamp_max, int32_t *tmp,
                             hipStream_t stream, int64_t *total64_out)
{
    if (n <= 0) return PCCNN_OK;
    if (n <= SCAN_SMALL_MAX) {
        long long *total = (long long *)total64_out;
        if (n <= 4 * SCAN_SMALL_THREADS) scan_small_kernel<4><<<1, SCAN_SMALL_THREADS, 0, stream>>>(in, out, n, clamp_max, total);
        else if (n <= 8 * SCAN_SMALL_THREADS) scan_small_kernel<8><<<1, SCAN_SMALL_THREADS, 0, stream>>>(in, out, n, clamp_max, total);
        else if (n <= 16 * SCAN_SMALL_THREADS) scan_small_kernel<16><<<1, SCAN_SMALL_THREADS, 0, stream>>>(in, out, n, clamp_max, total);
        else if (n <= 32 * SCAN_SMALL_THREADS) scan_small_kernel<32><<<1, SCAN_SMALL_THREADS, 0, stream>>>(in, out, n, clamp_max, total);
        else scan_small_kernel<48><<<1, SCAN_SMALL_THREADS, 0, stream>>>(in, out, n, clamp_max, total);
        PCCNN_LAUNCH_CHECK();
        return PCCNN_OK;
    }
    int64_t tiles = pccnn_ceil_div(n, SCAN_TILE);
    // 64-bit tile sums behind the 32-bit ones (8-byte aligned); with a single tile its sum is the total
    long long *sums64 = nullptr;
    if (total64_out) sums64 = tiles > 1 ? (long long *)(tmp + 2 * ((tiles + 2) / 2)) : (long long *)total64_out;
    scan_tiles_kernel<<<(unsigned)tiles, SCAN_THREADS, 0, stream>>>(in, out, n, clamp_max, tmp, sums64);
    PCCNN_LAUNCH_CHECK();
    if (tiles > 1) {
        scan_tile_sums_kernel<<<1, SCAN_THREADS, 0, stream>>>(tmp, tiles, sums64, (long long *)total64_out);
        PCCNN_LAUNCH_CHECK();
        scan_add_kernel<<<(unsigned)tiles, SCAN_THREADS, 0, stream>>>(out, n, tmp);
        PCCNN_LAUNCH_CHECK();
    }
    return PCCNN_OK;
}
