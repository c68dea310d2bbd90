// Shared host/device helpers of libpccnn_hip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/pccnn_hip.h"

#define PCCNN_WAVE 64
#define PCCNN_MAX_DIMS 6                                // point dimensions handled: 2 .. 6, as the reference's tests use

// KERNEL<D> LAUNCH for the run-time dimension d (2 .. 6), e.g.
//   PCCNN_DIM_DISPATCH(d, my_kernel, <<<grid, block, 0, stream>>>(args));
#define PCCNN_DIM_DISPATCH(d, KERNEL, ...)                                               \
    do {                                                                                 \
        switch (d) {                                                                     \
        case 2: KERNEL<2> __VA_ARGS__; break;                                              \
        case 3: KERNEL<3> __VA_ARGS__; break;                                              \
        case 4: KERNEL<4> __VA_ARGS__; break;                                              \
        case 5: KERNEL<5> __VA_ARGS__; break;                                              \
        default: KERNEL<6> __VA_ARGS__; break;                                             \
        }                                                                                \
    } while (0)

void pccnn_set_error(const char *fmt, ...);

#define PCCNN_REQUIRE(cond, code, ...)                                                   \
    do {                                                                                 \
        if (!(cond)) {                                                                   \
            pccnn_set_error(__VA_ARGS__);                                                \
            return (code);                                                               \
        }                                                                                \
    } while (0)

#define PCCNN_HIP_CHECK(expr)                                                            \
    do {                                                                                 \
        hipError_t err__ = (expr);                                                       \
        if (err__ != hipSuccess) {                                                       \
            pccnn_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(err__), __FILE__, __LINE__); \
            return PCCNN_ERR_HIP;                                                        \
        }                                                                                \
    } while (0)

#define PCCNN_LAUNCH_CHECK() PCCNN_HIP_CHECK(hipGetLastError())

static inline int64_t pccnn_ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t pccnn_align(size_t x) { return (x + 255) & ~(size_t)255; }

// Carves 256-byte aligned pieces out of a caller-provided workspace.
struct PccnnArena {
    char *base;
    size_t size, used;
    PccnnArena(void *p, size_t s) : base((char *)p), size(s), used(0) {}
    template <typename T> T *take(size_t count)
    {
        size_t bytes = pccnn_align(count * sizeof(T));
        if (base == nullptr || used + bytes > size) { used = size + 1; return nullptr; }
        T *r = (T *)(base + used);
        used += bytes;
        return r;
    }
    bool ok() const { return used <= size; }
};

#ifdef __HIPCC__
__device__ __forceinline__ int pccnn_lane() { return (int)__lane_id(); }

__device__ __forceinline__ unsigned long long pccnn_lanemask_lt()
{
    return (1ull << pccnn_lane()) - 1ull;
}

// Broadcast lane `src` (wave-uniform) of a 32-bit value to the whole wave.
__device__ __forceinline__ int pccnn_bcast_i(int v, int src)
{
    return __builtin_amdgcn_readlane(v, __builtin_amdgcn_readfirstlane(src));
}
__device__ __forceinline__ float pccnn_bcast_f(float v, int src)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), __builtin_amdgcn_readfirstlane(src)));
}
__device__ __forceinline__ long long pccnn_bcast_ll(long long v, int src)
{
    int lo = pccnn_bcast_i((int)(v & 0xffffffffll), src);
    int hi = pccnn_bcast_i((int)(v >> 32), src);
    return ((long long)hi << 32) | (unsigned int)lo;
}

// fp32 -> bf16 bit pattern, round to nearest even; a NaN stays a (quiet) NaN.
__device__ __forceinline__ uint16_t pccnn_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float pccnn_wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
#endif

// Optional per-kernel timing (off by default): a PccnnTimed object brackets the launches made
// during its lifetime with two events on the launch stream; pccnn_timing_read sums them up.
enum PccnnTimerId {
    PCCNN_T_GEMM = 0, PCCNN_T_PROJ_FWD, PCCNN_T_PROJ_BWD, PCCNN_T_BASIS_BWD, PCCNN_T_NB_COUNT, PCCNN_T_NB_FILL,
    PCCNN_T_SORT, PCCNN_T_KEYS, PCCNN_T_GRID, PCCNN_T_PDF, PCCNN_T_SCAN, PCCNN_T_COUNT
};
struct PccnnTimed {
    int id;
    hipStream_t stream;
    hipEvent_t stop;
    bool on;
    PccnnTimed(int id, hipStream_t s);
    ~PccnnTimed();
};

// Device-wide inclusive scan of int32 (scan.hip).  `clamp_max` > 0 clamps each input first.
// tmp must hold pccnn_scan_tmp_elems(n) ints.
size_t pccnn_scan_tmp_elems(int64_t n);
int pccnn_scan_inclusive_i32(const int32_t *in, int32_t *out, int64_t n, int clamp_max, int32_t *tmp,
                             hipStream_t stream);

// bf16 contraction (gemm_bf16.hip), used by conv.hip.
extern "C" int pccnn_f32_to_bf16(const float *src, uint16_t *dst, int64_t count, void *stream);
extern "C" int pccnn_gemm_bf16(const uint16_t *a, const uint16_t *b, float *c, int64_t rows, int64_t cols,
                               int64_t inner, int a_trans, int b_trans, int64_t lda, int64_t ldb, int64_t ldc,
                               int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, int split_k,
                               void *workspace, size_t workspace_bytes, void *stream);

// Internal sort entry used by other translation units.
int pccnn_fill_i32(int32_t *p, int32_t value, int64_t count, hipStream_t stream);
int pccnn_fill_f32(float *p, float value, int64_t count, hipStream_t stream);
