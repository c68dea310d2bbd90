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

// ---- sums over groups of lanes without going through the LDS crossbar ----------------------------------------
// A wavefront is four rows of sixteen lanes.  Inside a row, data-parallel-primitive operands (quad permutes, row
// rotations, mirrors) come for free with the add; between rows, gfx950's row swaps (v_permlane16_swap: odd rows of
// the first operand <-> even rows of the second; v_permlane32_swap: upper half of the first <-> lower half of the
// second) exchange whole rows in one instruction.  All lanes must be active.
template <int CTRL>
__device__ __forceinline__ float pccnn_dpp(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
#define PCCNN_DPP_QUAD_XOR1 0xb1      // quad_perm [1,0,3,2]
#define PCCNN_DPP_QUAD_XOR2 0x4e      // quad_perm [2,3,0,1]
#define PCCNN_DPP_ROW_ROR(n) (0x120 + (n))
#define PCCNN_DPP_ROW_MIRROR 0x140
#define PCCNN_DPP_ROW_HALF_MIRROR 0x141

// Inclusive prefix sum over the 64 lanes of a wavefront, all of them active: shifts by 1, 2, 4 and 8 inside the
// rows of sixteen (a lane whose source falls outside its row adds zero), then lane 15 of a row broadcast into the
// next row (rows 1 and 3), then lane 31 into the upper half - six adds whose second operand comes with the
// instruction, where six __shfl_up go through the LDS crossbar one after the other.
__device__ __forceinline__ int pccnn_wave_inclusive_scan_i(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);     // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);     // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);     // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);     // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);     // row_bcast:15, rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);     // row_bcast:31, rows 2 and 3
    return v;
}

// v + (v of the row 16 lanes away), in every lane: rows {0,1} and {2,3} are paired.
__device__ __forceinline__ float pccnn_add_row_xor16(float v)
{
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// v + (v of the lane 32 away), in every lane.
__device__ __forceinline__ float pccnn_add_row_xor32(float v)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Sum over each aligned group of WIDTH consecutive lanes (WIDTH a power of two, 1..64), left in every lane of the
// group.  The mirrors act as exchanges with the other half because the halves are uniform by then.
template <int WIDTH>
__device__ __forceinline__ float pccnn_group_sum(float v)
{
    if (WIDTH >= 2) v += pccnn_dpp<PCCNN_DPP_QUAD_XOR1>(v);
    if (WIDTH >= 4) v += pccnn_dpp<PCCNN_DPP_QUAD_XOR2>(v);
    if (WIDTH >= 8) v += pccnn_dpp<PCCNN_DPP_ROW_HALF_MIRROR>(v);
    if (WIDTH >= 16) v += pccnn_dpp<PCCNN_DPP_ROW_MIRROR>(v);
    if (WIDTH >= 32) v = pccnn_add_row_xor16(v);
    if (WIDTH >= 64) v = pccnn_add_row_xor32(v);
    return v;
}

// Minimum (MAX = false) or maximum over the 64 lanes of a wavefront, left in every lane; the exchanges of
// pccnn_group_sum<64>.  All lanes must be active.
template <bool MAX>
__device__ __forceinline__ float pccnn_wave_minmax(float v)
{
    auto pick = [](float a, float b) { return MAX ? fmaxf(a, b) : fminf(a, b); };
    v = pick(v, pccnn_dpp<PCCNN_DPP_QUAD_XOR1>(v));
    v = pick(v, pccnn_dpp<PCCNN_DPP_QUAD_XOR2>(v));
    v = pick(v, pccnn_dpp<PCCNN_DPP_ROW_HALF_MIRROR>(v));
    v = pick(v, pccnn_dpp<PCCNN_DPP_ROW_MIRROR>(v));
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = pick(__uint_as_float(r[0]), __uint_as_float(r[1]));
    const auto q = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return pick(__uint_as_float(q[0]), __uint_as_float(q[1]));
}

// Sum over the lanes that share (lane % STRIDE) (STRIDE a power of two, 1..64), left in every one of them.
// Inside a row the cosets are closed under rotation, so rotations by STRIDE, 2 STRIDE, ... add them up.
template <int STRIDE>
__device__ __forceinline__ float pccnn_strided_sum(float v)
{
    if (STRIDE <= 1) v += pccnn_dpp<PCCNN_DPP_ROW_ROR(1)>(v);
    if (STRIDE <= 2) v += pccnn_dpp<PCCNN_DPP_ROW_ROR(2)>(v);
    if (STRIDE <= 4) v += pccnn_dpp<PCCNN_DPP_ROW_ROR(4)>(v);
    if (STRIDE <= 8) v += pccnn_dpp<PCCNN_DPP_ROW_ROR(8)>(v);
    if (STRIDE <= 16) v = pccnn_add_row_xor16(v);
    if (STRIDE <= 32) v = pccnn_add_row_xor32(v);
    return v;
}

// Four values, each to be summed over the four rows (lanes l, l + 16, l + 32, l + 48): three row swaps and three
// adds do all four at once.  On return the lanes of row r hold the sum of value pccnn_rows4_slot(r).
__device__ __forceinline__ float pccnn_rows4_sum(float a0, float a1, float a2, float a3)
{
    const auto p = __builtin_amdgcn_permlane32_swap(__float_as_uint(a0), __float_as_uint(a1), false, false);
    const auto q = __builtin_amdgcn_permlane32_swap(__float_as_uint(a2), __float_as_uint(a3), false, false);
    // rows of u: a0(r0+r2), a0(r1+r3), a1(r0+r2), a1(r1+r3); v likewise for a2, a3
    const float u = __uint_as_float(p[0]) + __uint_as_float(p[1]);
    const float v = __uint_as_float(q[0]) + __uint_as_float(q[1]);
    const auto w = __builtin_amdgcn_permlane16_swap(__float_as_uint(u), __float_as_uint(v), false, false);
    return __uint_as_float(w[0]) + __uint_as_float(w[1]);          // rows: a0, a2, a1, a3
}
__device__ __forceinline__ int pccnn_rows4_slot(int row) { return ((row & 1) << 1) | (row >> 1); }

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
// A negative id never times (and so never creates an event).
enum PccnnTimerId {
    PCCNN_T_GEMM = 0, PCCNN_T_PROJ_FWD, PCCNN_T_PROJ_BWD, PCCNN_T_BASIS_BWD, PCCNN_T_NB_COUNT, PCCNN_T_NB_FILL,
    PCCNN_T_SORT, PCCNN_T_KEYS, PCCNN_T_GRID, PCCNN_T_PDF, PCCNN_T_SCAN, PCCNN_T_FUSED_FWD, PCCNN_T_COUNT
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
// total64_out (nullable, device): the grand total without the 32-bit wrap-around.
int pccnn_scan_inclusive_i32(const int32_t *in, int32_t *out, int64_t n, int clamp_max, int32_t *tmp,
                             hipStream_t stream, int64_t *total64_out = nullptr);

// bf16 contraction (gemm_bf16.hip), used by conv.hip.
extern "C" int pccnn_f32_to_bf16(const float *src, uint16_t *dst, int64_t count, void *stream);
extern "C" int pccnn_gemm_bf16(const uint16_t *a, const uint16_t *b, float *c, int64_t rows, int64_t cols,
                               int64_t inner, int a_trans, int b_trans, int64_t lda, int64_t ldb, int64_t ldc,
                               int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c, int split_k,
                               void *workspace, size_t workspace_bytes, void *stream);

// A grid size by value (kernel argument), and the key computation that takes it that way (keys_grid.hip).
struct PccnnGridDims {
    int v[PCCNN_MAX_DIMS];
};
int pccnn_compute_keys_sized(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                             const int32_t *num_cells_host, const float *cell_size, int64_t n, int d,
                             int32_t *num_cells_out, int64_t *keys_out, hipStream_t stream);
// Workgroups are handed to the 8 XCDs round-robin by their linear id, and each XCD has its own L2.  A kernel whose
// consecutive workgroups work on neighboring parts of space (sorted samples sharing their neighbors) launches
// pccnn_xcd_grid(blocks, chunk) workgroups and lets workgroup b do the work of logical block
// pccnn_xcd_block(b, grid, chunk): runs of `chunk` consecutive logical blocks go to one XCD, so that what
// neighbors share stays in its L2, and the runs are dealt to the XCDs in turn, so that all of them sweep through
// the same part of space at a time and a dense region does not land on one XCD alone.  A grid of fewer than
// 8 * chunk blocks is cut into eight runs.  Logical blocks past the real count must return at once.
#define PCCNN_XCDS 8
static inline unsigned pccnn_xcd_grid(int64_t blocks, int chunk)
{
    int64_t per = (blocks + PCCNN_XCDS - 1) / PCCNN_XCDS;
    if (per > chunk) per = chunk;
    if (per < 1) per = 1;
    const int64_t super = per * PCCNN_XCDS;
    return (unsigned)(((blocks + super - 1) / super) * super);
}
#ifdef __HIPCC__
__device__ __forceinline__ int64_t pccnn_xcd_block(unsigned block, unsigned grid, int chunk)
{
    const unsigned per = grid / PCCNN_XCDS < (unsigned)chunk ? grid / PCCNN_XCDS : (unsigned)chunk;
    const unsigned super = per * PCCNN_XCDS;
    const unsigned within = block % super;
    return (int64_t)(block - within) + (int64_t)(within % PCCNN_XCDS) * per + within / PCCNN_XCDS;
}
#endif

// The bounding box of a subset of a sorted cloud, and a second copy of the result for one read-back.  With
// `selected`, point i counts only when selected[i] != 0; with `perm`, its cloud is batch_ids[perm[i]] (the points
// are a sorted copy, the cloud ids are not).  With `tail`, the padded boxes are also written there as
// [minima | maxima] followed by the 32-bit word at `count_src` (or 1), so that one copy brings box and count to the
// host - or none, when `tail` is host memory mapped into the device's address space: the word is written last, so
// the host can poll it (at most 256 box values then: the kernel that pads the boxes must be one workgroup).
struct PccnnBoxMask {
    const int32_t *selected = nullptr;
    const int32_t *perm = nullptr;
    float *tail = nullptr;
    const int32_t *count_src = nullptr;
#ifdef __HIPCC__
    __device__ __forceinline__ int cloud_of(const int32_t *__restrict__ batch_ids, int64_t i) const
    {
        if (selected != nullptr && selected[i] == 0) return -1;
        return batch_ids[perm != nullptr ? (int64_t)perm[i] : i];
    }
    __device__ __forceinline__ void second_copy(int i, int count, float lo, float hi) const
    {
        if (tail == nullptr) return;
        tail[i] = lo;
        tail[count + i] = hi;
    }
    // The word behind the boxes, written by one thread after every box value of `tail` has left (the kernels call
    // this behind a system-scope fence and a workgroup barrier, so a host that polls the word in mapped memory
    // finds the boxes complete): the 32-bit word at `count_src`, or 1 without one.
    __device__ __forceinline__ void publish(int count) const
    {
        if (tail != nullptr) ((volatile int32_t *)tail)[2 * count] = count_src != nullptr ? *count_src : 1;
    }
#endif
};
int pccnn_bounding_box_masked(const float *pts, const int32_t *batch_ids, int64_t n, int d, int batch_size,
                              float *aabb_min_out, float *aabb_max_out, const PccnnBoxMask &mask, void *stream);

// Where the next pccnn_find_neighbors_count of this host thread writes its 64-bit pair total instead of the head of
// its workspace (device-visible memory, e.g. mapped host memory; nullptr: the workspace again).
void pccnn_redirect_pair_total(int64_t *destination);

// Where the keys of a sort come from when they are made on the way in (3-D points): the arguments of the key
// computation.  The grid size is read from `num_cells` (device) or, with `use_sized`, taken from `sized` and written
// to `num_cells_out` for the kernels that follow.
struct PccnnKeySource {
    const float *pts;
    const int32_t *batch_ids;
    const float *aabb_min;
    const float *cell_size;
    const int32_t *num_cells;
    PccnnGridDims sized;
    int32_t *num_cells_out;
    int use_sized;
};
// pccnn_compute_keys (3-D) and pccnn_sort_keys in one: the first histogram pass computes the keys (sort.hip).
int pccnn_sort_keys_from_points(const PccnnKeySource &source, int64_t *keys_out, int64_t n, int key_bits,
                                int64_t *sorted_keys_out, int32_t *perm_out, float *sorted_pts_out, void *workspace,
                                size_t workspace_bytes, void *stream);
#ifdef __HIPCC__
// The cell key of 3-D point i: fp32, exactly in this order - subtract the box corner, multiply by the fp32
// reciprocal of the cell size, floor, clamp (no fused multiply-add).
__device__ __forceinline__ long long pccnn_point_key3(const float *__restrict__ pts, const int32_t *__restrict__ batch_ids,
                                                      const float *__restrict__ aabb_min,
                                                      const float *__restrict__ cell_size, const int (&nc)[3], int64_t i)
{
#pragma clang fp contract(off)
    const int b = batch_ids[i];
    long long key = 0, accum = 1;
#pragma unroll
    for (int k = 2; k >= 0; --k) {
        const float inv = __fdiv_rn(1.0f, cell_size[k]);
        const float rel = (pts[i * 3 + k] - aabb_min[(int64_t)b * 3 + k]) * inv;
        int c = (int)floorf(rel);
        c = max(0, min(c, nc[k] - 1));
        key += (long long)c * accum;
        accum *= nc[k];
    }
    return key + accum * (long long)b;
}
#endif
int pccnn_grid_build_sized3(const float *pts, const int32_t *batch_ids, const float *aabb_min,
                            const int32_t *num_cells_host, const float *cell_size, int64_t n, int key_bits,
                            int64_t num_pillars, int64_t total_cells, int32_t *num_cells_out, int64_t *keys_out,
                            int64_t *sorted_keys_out, int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out,
                            int32_t *cell_table_out, void *workspace, size_t workspace_bytes, void *stream);
// The rest of pccnn_grid_build after the keys: sort, pillar table, cell table (keys_grid.hip).
int pccnn_grid_build_from_keys(const int64_t *keys, const float *pts, const int32_t *num_cells, int64_t n, int d,
                               int key_bits, int64_t num_pillars, int64_t total_cells, int64_t *sorted_keys_out,
                               int32_t *perm_out, float *sorted_pts_out, int32_t *grid_ds_out, int32_t *cell_table_out,
                               void *workspace, size_t workspace_bytes, void *stream);

// Internal sort entry used by other translation units.
int pccnn_fill_i32(int32_t *p, int32_t value, int64_t count, hipStream_t stream);
int pccnn_fill_f32(float *p, float value, int64_t count, hipStream_t stream);
