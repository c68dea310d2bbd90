// Radius neighbor search on the pillar grid: count pass, device scan, fill pass.
//
// One wavefront owns a tile of 64 consecutive samples of `sample_order` (key order when the
// caller provides it), one sample per lane.  Every lane decodes its own cell, looks up the
// 3 x 3 pillar walk of that cell (two reads of the cell start table per pillar, or two binary
// searches in the pillar's slice of the sorted keys) and parks the non-empty index ranges in LDS.
// The lanes then walk their own candidate lists side by side, a few candidates per lane and
// iteration: neighbouring lanes sit in the same or adjacent cells, so their loads of the sorted
// points fall into the same few cache lines.  The fill pass repeats the walk over 16-byte
// (x, y, z, output id) records packed beforehand and stores the hits straight into the sample's
// segment, two pairs per store, in ascending sorted-point order, so no atomics are used and the
// output is deterministic.
#include "common.h"
#include "grid_walk.h"

// fp32 expressions in this file must round exactly as written (no fused multiply-add).
#pragma clang fp contract(off)

#define NB_THREADS 256
#define NB_WAVES (NB_THREADS / 64)
#define NB_UNROLL_COUNT 4                              // candidates per lane and iteration of the walk
#define NB_UNROLL_FILL 8
// The count pass of the one-lane walk can leave its decisions behind: bit 4 * i + u of a sample's mask is the
// outcome of candidate slot u of its walk iteration i (NB_UNROLL_COUNT slots per iteration).  Word w of all samples
// is one row, so the 64 lanes of a tile, which finish a word in the same iteration, store it as one run.
#define NB_PACK_FROM_PAIRS 1000000    // pairs from which the grouped fill packs its point records first
#ifndef NB_XCD_CHUNK
#define NB_XCD_CHUNK 64                    // consecutive workgroups of the walk kernels that share an XCD
#endif
#define NB_MASK_WORDS 16                               // 256 iterations = 1024 candidate slots per sample are recorded

struct NbArgs {
    const float *pts;          // sorted points [n,3]
    const int64_t *pt_keys;    // sorted keys [n]
    int64_t n;
    const float *samples;      // [m,3]
    const int64_t *sample_keys;
    int64_t m;
    const int32_t *order;      // nullable
    int presorted;             // samples / sample_keys are listed in `order` order already
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
    const float4 *rec;         // FILL: packed (x, y, z, id) of the sorted points
    unsigned long long *masks; // nullable: hit bits of the one-lane walk, [NB_MASK_WORDS][m_pad] (count writes, fill reads)
    int64_t m_pad;             // m rounded up to whole wavefronts
};

// Four consecutive ints at an 8-byte aligned address as one store instruction.
struct __attribute__((packed, aligned(8))) NbQuad { int v[4]; };
__device__ __forceinline__ void nb_store4(int *dst, int a0, int a1, int a2, int a3)
{
    NbQuad q;
    q.v[0] = a0; q.v[1] = a1; q.v[2] = a2; q.v[3] = a3;
    *reinterpret_cast<NbQuad *>(dst) = q;
}

// Index range [first, first + len) of the sorted points that lie in cells cmin..cmax of `pillar`.
__device__ __forceinline__ void nb_pillar_range(const NbArgs &a, long long pillar, int nc2, int cmin, int cmax,
                                                int &first, int &len)
{
    const GridRef g = {a.cell_table, a.total_cells, a.grid_ds, a.num_pillars, a.pt_keys, a.n};
    grid_pillar_range(g, pillar, nc2, cmin, cmax, first, len);
}

// rec[i] = (x, y, z, bits of the id to report for sorted point i): one aligned 16-byte load per candidate
// gives the fill pass the coordinates and the output id together.
__global__ void __launch_bounds__(256)
pack_points_kernel(const float *__restrict__ pts, const int32_t *__restrict__ remap, int64_t n,
                   float4 *__restrict__ rec)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float4 v;
    v.x = pts[i * 3 + 0];
    v.y = pts[i * 3 + 1];
    v.z = pts[i * 3 + 2];
    v.w = __int_as_float(remap ? remap[i] : (int)i);
    rec[i] = v;
}

// What a lane of the one-lane walk knows before it starts walking: its sample (index s, coordinates), and in
// ranges[wib][0 .. nr - 1][lane] the non-empty index ranges of the sorted points it has to look at.
struct NbLane {
    int lane, wib;
    int64_t base;
    bool live, valid;          // the wavefront has samples at all; this lane has one
    int s, nr;
    float sx, sy, sz, ir0, ir1, ir2;
};

__device__ __forceinline__ NbLane nb_lane_setup(const NbArgs &a, int2 (*ranges)[9][64])
{
    NbLane L;
    const int lane = pccnn_lane();
    const int wib = threadIdx.x >> 6;
    // (samples are walked in key order: an XCD gets one contiguous run of them)
    const int64_t wave = (pccnn_xcd_block(blockIdx.x, gridDim.x, NB_XCD_CHUNK) * NB_THREADS + threadIdx.x) >> 6;
    const int64_t base = wave * 64;
    L.live = base < a.m;                                       // wave-uniform
    if (!L.live) return L;
    const bool valid = base + lane < a.m;

    int s = 0;
    long long key = -1;
    float sx = 0.f, sy = 0.f, sz = 0.f;
    if (valid) {
        s = a.order ? a.order[base + lane] : (int)(base + lane);
        // entry of this sample in the sample arrays: its place in the walk order when the caller lists them
        // that way (coalesced reads), else its index (a gather)
        const int64_t at = a.presorted ? base + lane : (int64_t)s;
        key = a.sample_keys[at];
        sx = a.samples[at * 3 + 0];
        sy = a.samples[at * 3 + 1];
        sz = a.samples[at * 3 + 2];
    }
    const int nc0 = a.num_cells[0], nc1 = a.num_cells[1], nc2 = a.num_cells[2];
    const float ir0 = __fdiv_rn(1.0f, a.radii[0]);
    const float ir1 = __fdiv_rn(1.0f, a.radii[1]);
    const float ir2 = __fdiv_rn(1.0f, a.radii[2]);

    // key -> (pillar = (batch * nc0 + c0) * nc1 + c1, c0, c1, c2); 32-bit arithmetic when the whole tile allows it
    long long pil = 0;
    int c0 = 0, c1 = 0, c2 = 0;
    const bool usable = valid && key >= 0;
    if (__all(!usable || key < 0x7fffffffll)) {
        unsigned int k = usable ? (unsigned int)key : 0u;
        c2 = (int)(k % (unsigned int)nc2); k /= (unsigned int)nc2;
        c1 = (int)(k % (unsigned int)nc1); pil = k; k /= (unsigned int)nc1;
        c0 = (int)(k % (unsigned int)nc0);
    } else {
        long long k = usable ? key : 0;
        c2 = (int)(k % nc2); k /= nc2;
        c1 = (int)(k % nc1); pil = k; k /= nc1;
        c0 = (int)(k % nc0);
    }

    int nr = 0;
    if (usable) {
        const int cmin = c2 > 0 ? c2 - 1 : 0, cmax = c2 + 1 < nc2 ? c2 + 1 : nc2 - 1;
#pragma unroll
        for (int o = 0; o < 9; ++o) {
            const int dx = o / 3 - 1, dy = o % 3 - 1;
            const int x = c0 + dx, y = c1 + dy;
            if (x >= 0 && x < nc0 && y >= 0 && y < nc1) {
                int first, len;
                nb_pillar_range(a, pil + (long long)dx * nc1 + dy, nc2, cmin, cmax, first, len);
                if (len > 0) {
                    ranges[wib][nr][lane] = make_int2(first, len);
                    ++nr;
                }
            }
        }
    }

    L.lane = lane; L.wib = wib; L.base = base; L.valid = valid; L.s = s; L.nr = nr;
    L.sx = sx; L.sy = sy; L.sz = sz; L.ir0 = ir0; L.ir1 = ir1; L.ir2 = ir2;
    return L;
}

// OFF32 (count pass): the coordinate array is below 4 GiB, so a candidate's byte offset is a 32-bit number kept up
// to date with additions (one multiplication per range, none per candidate) and the loads take it beside a scalar
// base, instead of a 64-bit multiply-add per candidate.
template <bool FILL, bool CAPPED, int UNROLL, bool OFF32 = false>
__global__ void __launch_bounds__(NB_THREADS)
neighbors_kernel(NbArgs a)
{
    // ranges[w][r][lane] = r-th non-empty (first, len) range of the lane's sample; written and read by the
    // same lane only, so no barrier is involved
    __shared__ int2 ranges[NB_WAVES][9][64];

    const NbLane L = nb_lane_setup(a, ranges);
    if (!L.live) return;
    const int lane = L.lane, wib = L.wib, s = L.s, nr = L.nr;
    const int64_t base = L.base;
    const bool valid = L.valid;
    const float sx = L.sx, sy = L.sy, sz = L.sz, ir0 = L.ir0, ir1 = L.ir1, ir2 = L.ir2;

    unsigned int my_off = 0;                                    // FILL: next output slot of this lane's sample
    int raw = 0, take_step = 0;                                 // capped: see below
    if (FILL && valid) {
        my_off = s > 0 ? (unsigned int)a.ends[s - 1] : 0u;
        if (CAPPED) {
            raw = a.counts[s];
            take_step = raw < a.max_neighbors ? raw : a.max_neighbors;
        }
    }
    const unsigned int out_limit = FILL ? (unsigned int)a.t : 0u;
    int held = -1;                                              // FILL: a kept hit waiting for a partner

    // Capped samples keep hit number r (0-based, in walk order) iff floor((r+1)*cap/raw) > floor(r*cap/raw),
    // at slot floor(r*cap/raw): with err = (r*cap) mod raw this is "err + cap >= raw", and the slot advances by one
    // with every kept hit.  Samples at or below the cap use step = raw, which keeps every hit.
    int cnt = 0, err = 0;
    int r = 0, j = 0, first = 0, len = 0;
    // count, uncapped: the outcome of every candidate slot goes into the sample's mask (see NB_MASK_WORDS)
    const bool record = !FILL && UNROLL == NB_UNROLL_COUNT && a.masks != nullptr;
    unsigned long long word = 0ull;
    int it = 0;
    bool active = nr > 0;
    unsigned int byte_off = 0u;                                 // OFF32: 12 * (first + j)
    const char *const pts_bytes = (const char *)a.pts;
    if (active) {
        const int2 g = ranges[wib][0][lane];
        first = g.x;
        len = g.y;
        byte_off = 12u * (unsigned int)first;
    }
    while (__any(active)) {
        if (active) {
            // UNROLL consecutive candidates of the current range per iteration: their loads are issued
            // together; slots past the end of the range re-read its first candidate and are masked out
            const int idx = first + j;
            const int left = len - j;
            float px[UNROLL], py[UNROLL], pz[UNROLL];
            int id[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const int iu = idx + (u < left ? u : 0);
                if (FILL) {
                    const float4 v = a.rec[iu];
                    px[u] = v.x; py[u] = v.y; pz[u] = v.z;
                    id[u] = __float_as_int(v.w);
                } else if (OFF32) {
                    const float *q = (const float *)(pts_bytes + (byte_off + (u < left ? 12u * u : 0u)));
                    px[u] = q[0];
                    py[u] = q[1];
                    pz[u] = q[2];
                    id[u] = 0;
                } else {
                    px[u] = a.pts[(int64_t)iu * 3 + 0];
                    py[u] = a.pts[(int64_t)iu * 3 + 1];
                    pz[u] = a.pts[(int64_t)iu * 3 + 2];
                    id[u] = 0;
                }
            }
            unsigned int nibble = 0u;                               // count: the outcome of this iteration's slots
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                // fp32, no contraction: ((s - p) * (1/r)) squared, summed x, y, z; the reference tests
                // sqrt(acc) < 1, which for a correctly rounded fp32 sqrt holds exactly when acc < 1
                // (the largest float below 1 has a root below the midpoint to 1, so it rounds down).
                const float vx = (sx - px[u]) * ir0;
                const float vy = (sy - py[u]) * ir1;
                const float vz = (sz - pz[u]) * ir2;
                const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                if (u < left && acc < 1.0f) {
                    if (FILL) {
                        bool take = true;
                        if (CAPPED) {
                            err += take_step;
                            take = err >= raw;
                            if (take) err -= raw;
                        }
                        if (take) {
                            // kept hits leave in pairs: one 16-byte store per two pairs of the sample's segment
                            if (held < 0) {
                                held = id[u];
                            } else {
                                if (my_off + 1u < out_limit) {
                                    int *dst = a.neigh + 2 * (size_t)my_off;
                                    nb_store4(dst, held, s, id[u], s);
                                }
                                my_off += 2u;
                                held = -1;
                            }
                        }
                    }
                    if (FILL) ++cnt;
                    else nibble |= 1u << u;
                }
            }
            // one 64-bit shift and one population count per iteration, not one per slot
            if (!FILL) {
                word |= (unsigned long long)nibble << ((it & 15) << 2);
                cnt += __popc(nibble);
            }
            j += UNROLL;
            byte_off += 12u * UNROLL;
            if (j >= len) {
                j = 0;
                if (++r < nr) {
                    const int2 g = ranges[wib][r][lane];
                    first = g.x;
                    len = g.y;
                    byte_off = 12u * (unsigned int)first;
                } else {
                    active = false;
                }
            }
            if (!FILL) {
                ++it;
                // a word is complete after 16 iterations (for every lane still walking at once: one run of 8-byte
                // stores), or when the lane's walk ends
                if (record && ((it & 15) == 0 || !active) && ((it - 1) >> 4) < NB_MASK_WORDS) {
                    a.masks[(size_t)((it - 1) >> 4) * a.m_pad + base + lane] = word;
                    word = 0ull;
                }
            }
        }
    }
    if (FILL) {
        if (held >= 0 && my_off < out_limit) ((int2 *)a.neigh)[my_off] = make_int2(held, s);
    } else if (valid) {
        a.counts[s] = cnt;
    }
}

// The fill pass of the one-lane walk when the count pass has left its masks.  Nothing is tested again and no
// candidate is loaded: a lane reads its mask words (one run of 8-byte loads per word and tile), turns every set bit
// into the index of the sorted point it stands for - bit 4 i + u is slot u of walk iteration i, and the iterations
// of a sample are those of its ranges one after the other, ceil(len / 4) each -, fetches the ids of four neighbors
// at a time and writes two pairs per store.  A pass over a word depends on memory once per four neighbors, where
// the walk depended on it once per iteration.  Beyond the NB_MASK_WORDS * 16 recorded iterations (a sample with
// more than about 1000 candidates) the lane tests the remaining candidates itself, exactly as the count pass did.
__global__ void __launch_bounds__(NB_THREADS)
neighbors_fill_masks_kernel(NbArgs a)
{
    __shared__ int2 ranges[NB_WAVES][9][64];
    __shared__ __attribute__((aligned(16))) int stage_ids[NB_WAVES][64][8];
    __shared__ int4 stage_meta[NB_WAVES][64];
    const NbLane L = nb_lane_setup(a, ranges);
    if (!L.live) return;
    const int lane = L.lane, wib = L.wib, s = L.s, nr = L.nr;
    const int64_t base = L.base;

    unsigned int my_off = 0;
    if (L.valid) my_off = s > 0 ? (unsigned int)a.ends[s - 1] : 0u;
    const unsigned int out_limit = (unsigned int)a.t;

    int total_it = 0;                                           // iterations of this lane's walk
    for (int q = 0; q < nr; ++q) total_it += (ranges[wib][q][lane].y + NB_UNROLL_COUNT - 1) / NB_UNROLL_COUNT;
    // the range the enumeration stands in: its first iteration, its number of iterations, its first point
    int r = 0, cum = 0, nit = 0, first = 0;
    if (nr > 0) {
        const int2 g = ranges[wib][0][lane];
        first = g.x;
        nit = (g.y + NB_UNROLL_COUNT - 1) / NB_UNROLL_COUNT;
    }
    const int my_words = total_it < NB_MASK_WORDS * 16 ? (total_it + 15) >> 4 : NB_MASK_WORDS;
    int w = 0;
    unsigned long long word = my_words > 0 ? a.masks[base + lane] : 0ull;
    unsigned long long next_word = my_words > 1 ? a.masks[(size_t)a.m_pad + base + lane] : 0ull;
    // Up to eight neighbors per round, and never across a 64-byte boundary of the pair list: after its first
    // round a lane writes whole aligned 64-byte pieces of its segment, four 16-byte stores back to back, so a
    // piece reaches memory complete instead of in quarters that leave the L2 one by one.
    while (__any(word != 0ull || w + 1 < my_words)) {
        const int cap = 8 - (int)(my_off & 7u);
        int idx[8], have = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            idx[q] = 0;
            while (word == 0ull && w + 1 < my_words) {          // on to the lane's next word that has a bit set:
                ++w;                                            // the neighbors of a round stay in slots 0 .. have - 1
                word = next_word;
                if (w + 1 < my_words) next_word = a.masks[(size_t)(w + 1) * a.m_pad + base + lane];
            }
            if (have < cap && word != 0ull) {
                const int b = __builtin_ctzll(word);
                word &= word - 1ull;
                const int i = (w << 4) + (b >> 2);
                while (i >= cum + nit && r + 1 < nr) {          // at most nr - 1 steps in the life of the lane
                    cum += nit;
                    ++r;
                    const int2 g = ranges[wib][r][lane];
                    first = g.x;
                    nit = (g.y + NB_UNROLL_COUNT - 1) / NB_UNROLL_COUNT;
                }
                // (masks that no count call wrote cannot send a lane out of its ranges or out of the points)
                const int at = first + ((i - cum) << 2) + (b & 3);
                idx[q] = (i < cum + nit && (int64_t)at < a.n) ? at : 0;
                have = q + 1;
            }
        }
        int id[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) id[q] = (q < have && a.remap) ? a.remap[idx[q]] : idx[q];
        // The round's pieces leave through LDS: every lane parks its (up to) eight ids and where they go, then four
        // adjacent lanes write one lane's piece, 16 bytes each, so that a 64-byte piece reaches the memory system as
        // one request from one instruction instead of as four quarters from four.
        *(int4 *)&stage_ids[wib][lane][0] = make_int4(id[0], id[1], id[2], id[3]);
        *(int4 *)&stage_ids[wib][lane][4] = make_int4(id[4], id[5], id[6], id[7]);
        stage_meta[wib][lane] = make_int4((int)my_off, have, s, 0);
        // (a wavefront's own LDS writes are in order with its reads)
#pragma unroll
        for (int part = 0; part < 4; ++part) {
            const int owner = part * 16 + (lane >> 2), j = lane & 3;
            const int4 m = stage_meta[wib][owner];
            const int2 two = *(const int2 *)&stage_ids[wib][owner][2 * j];
            const unsigned int at = (unsigned int)m.x + 2u * (unsigned int)j;
            if (2 * j + 1 < m.y) {
                if (at + 1u < out_limit) nb_store4(a.neigh + 2 * (size_t)at, two.x, m.z, two.y, m.z);
            } else if (2 * j < m.y) {
                if (at < out_limit) ((int2 *)a.neigh)[at] = make_int2(two.x, m.z);
            }
        }
        my_off += (unsigned int)have;
    }
    int held = -1;
    auto emit = [&](int id) {
        if (held < 0) {
            held = id;
        } else {
            if (my_off + 1u < out_limit) nb_store4(a.neigh + 2 * (size_t)my_off, held, s, id, s);
            my_off += 2u;
            held = -1;
        }
    };
    // the rare tail: iterations that the masks do not cover
    if (__any(total_it > NB_MASK_WORDS * 16)) {
        bool active = total_it > NB_MASK_WORDS * 16;
        int j = 0, len = 0;
        if (active) {
            const int it0 = NB_MASK_WORDS * 16;
            while (it0 >= cum + nit && r + 1 < nr) {
                cum += nit;
                ++r;
                nit = (ranges[wib][r][lane].y + NB_UNROLL_COUNT - 1) / NB_UNROLL_COUNT;
            }
            const int2 g = ranges[wib][r][lane];
            first = g.x;
            len = g.y;
            j = (it0 - cum) * NB_UNROLL_COUNT;
        }
        while (__any(active)) {
            if (active) {
                const int left = len - j;
                float px[NB_UNROLL_COUNT], py[NB_UNROLL_COUNT], pz[NB_UNROLL_COUNT];
                int id[NB_UNROLL_COUNT];
#pragma unroll
                for (int u = 0; u < NB_UNROLL_COUNT; ++u) {         // all loads of the iteration together
                    const int64_t iu = first + j + (u < left ? u : 0);
                    px[u] = a.pts[iu * 3 + 0];
                    py[u] = a.pts[iu * 3 + 1];
                    pz[u] = a.pts[iu * 3 + 2];
                    id[u] = a.remap ? a.remap[iu] : (int)iu;
                }
#pragma unroll
                for (int u = 0; u < NB_UNROLL_COUNT; ++u) {
                    const float vx = (L.sx - px[u]) * L.ir0;
                    const float vy = (L.sy - py[u]) * L.ir1;
                    const float vz = (L.sz - pz[u]) * L.ir2;
                    const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                    if (u < left && acc < 1.0f) emit(id[u]);
                }
                j += NB_UNROLL_COUNT;
                if (j >= len) {
                    j = 0;
                    if (++r < nr) {
                        const int2 g = ranges[wib][r][lane];
                        first = g.x;
                        len = g.y;
                    } else {
                        active = false;
                    }
                }
            }
        }
    }
    if (held >= 0 && my_off < out_limit) ((int2 *)a.neigh)[my_off] = make_int2(held, s);
}

// Few samples against many points (every pooling level of a hierarchy): with one sample per lane the launch has
// too few wavefronts and every lane a long walk.  Here G lanes share a sample: lane 0..8 of the group look up the
// nine pillar ranges, then the group strides over every range together, one candidate per lane and step; a ballot
// over the group's lanes counts the hits of the step and ranks them, so the pairs of a sample still come out in
// ascending sorted-point order, without atomics.  The capped subset is the same as in the one-lane walk: hit
// number r is kept iff floor((r + 1) cap / raw) > floor(r cap / raw), at slot floor(r cap / raw).
template <bool FILL, bool CAPPED, int G>
__global__ void __launch_bounds__(NB_THREADS)
neighbors_group_kernel(NbArgs a)
{
    constexpr int GROUPS = 64 / G;                              // samples per wavefront
    __shared__ int2 ranges[NB_WAVES][GROUPS][9];
    const int lane = pccnn_lane();
    const int wib = threadIdx.x >> 6;
    const int grp = lane / G, sub = lane % G;
    // (samples are walked in key order: an XCD gets one contiguous run of them)
    const int64_t wave = (pccnn_xcd_block(blockIdx.x, gridDim.x, NB_XCD_CHUNK) * NB_THREADS + threadIdx.x) >> 6;
    const int64_t at0 = wave * GROUPS + grp;                    // place of the group's sample in the walk order
    if (wave * GROUPS >= a.m) return;                           // wave-uniform
    const bool valid = at0 < a.m;

    int s = 0;
    long long key = -1;
    float sx = 0.f, sy = 0.f, sz = 0.f;
    if (valid) {
        s = a.order ? a.order[at0] : (int)at0;
        const int64_t at = a.presorted ? at0 : (int64_t)s;
        key = a.sample_keys[at];
        sx = a.samples[at * 3 + 0];
        sy = a.samples[at * 3 + 1];
        sz = a.samples[at * 3 + 2];
    }
    const int nc0 = a.num_cells[0], nc1 = a.num_cells[1], nc2 = a.num_cells[2];
    const float ir0 = __fdiv_rn(1.0f, a.radii[0]);
    const float ir1 = __fdiv_rn(1.0f, a.radii[1]);
    const float ir2 = __fdiv_rn(1.0f, a.radii[2]);
    const bool usable = valid && key >= 0;
    long long k = usable ? key : 0;
    const int c2 = (int)(k % nc2); k /= nc2;
    const int c1 = (int)(k % nc1);
    const long long pil = k; k /= nc1;
    const int c0 = (int)(k % nc0);
    // the nine ranges, in pillar order (ascending sorted index); lane o of the group looks up range o
    for (int o = sub; o < 9; o += G) {
        int first = 0, len = 0;
        if (usable) {
            const int cmin = c2 > 0 ? c2 - 1 : 0, cmax = c2 + 1 < nc2 ? c2 + 1 : nc2 - 1;
            const int dx = o / 3 - 1, dy = o % 3 - 1;
            const int x = c0 + dx, y = c1 + dy;
            if (x >= 0 && x < nc0 && y >= 0 && y < nc1)
                nb_pillar_range(a, pil + (long long)dx * nc1 + dy, nc2, cmin, cmax, first, len);
        }
        ranges[wib][grp][o] = make_int2(first, len);
    }
    // (a wavefront's own LDS writes are in order with its reads: no barrier between the lanes of a group)

    unsigned int seg = 0;                                       // FILL: first output slot of the sample
    long long raw = 0, cap = 0;
    if (FILL && valid) {
        seg = s > 0 ? (unsigned int)a.ends[s - 1] : 0u;
        if (CAPPED) {
            raw = a.counts[s];
            cap = raw < a.max_neighbors ? raw : a.max_neighbors;
        }
    }
    const unsigned int out_limit = FILL ? (unsigned int)a.t : 0u;
    const unsigned long long group_bits = (G == 64) ? ~0ull : (((1ull << (G & 63)) - 1ull) << (grp * G));
    const unsigned long long below = group_bits & pccnn_lanemask_lt();

    int cnt = 0;                                                // hits of the sample so far (same in all its lanes)
    int r = 0, j0 = 0;
    int2 cur = ranges[wib][grp][0];
    bool active = usable;
    while (__any(active)) {
        bool hit = false;
        int id = 0;
        if (active) {
            const int j = j0 + sub;
            if (j < cur.y) {
                const int idx = cur.x + j;
                float px, py, pz;
                if (FILL && a.rec != nullptr) {
                    const float4 v = a.rec[idx];
                    px = v.x; py = v.y; pz = v.z;
                    id = __float_as_int(v.w);
                } else {
                    // (count, and the fill of a small search, where packing the records would be one more launch)
                    px = a.pts[(int64_t)idx * 3 + 0];
                    py = a.pts[(int64_t)idx * 3 + 1];
                    pz = a.pts[(int64_t)idx * 3 + 2];
                    if (FILL) id = a.remap ? a.remap[idx] : idx;
                }
                // fp32, no contraction: the predicate of the one-lane walk
                const float vx = (sx - px) * ir0;
                const float vy = (sy - py) * ir1;
                const float vz = (sz - pz) * ir2;
                const float acc = ((0.0f + vx * vx) + vy * vy) + vz * vz;
                hit = acc < 1.0f;
            }
        }
        const unsigned long long hits = __ballot(hit);
        if (active) {
            if (FILL && hit) {
                const long long rank = cnt + __popcll(hits & below);        // number of this hit in walk order
                bool take = true;
                long long slot = rank;
                if (CAPPED) {
                    slot = rank * cap / raw;
                    take = (rank + 1) * cap / raw > slot;
                }
                const unsigned long long at = (unsigned long long)seg + (unsigned long long)slot;
                if (take && at < out_limit) ((int2 *)a.neigh)[at] = make_int2(id, s);
            }
            cnt += __popcll(hits & group_bits);
            j0 += G;
            if (j0 >= cur.y) {
                j0 = 0;
                if (++r < 9) cur = ranges[wib][grp][r];
                else active = false;
            }
        }
    }
    if (!FILL && valid && sub == 0) a.counts[s] = cnt;
}

#define NB_CHIP_LANES (256 * 32 * 64)       // lanes of one round of wavefronts at full occupancy

// Lanes per sample: one when there are about as many samples as points, more when the samples are few.
static int nb_group_size(int64_t n, int64_t m, int d)
{
    if (d != 3 || m <= 0) return 1;
    if (n >= 16 * m) return 64;
    if (n >= 4 * m) return 16;
    // about as many samples as points, but few of them: one sample per lane leaves the chip short of wavefronts
    // (65 536 samples are 4 per CU), so lanes share a sample as long as the launch still fits the chip in one round
    // of 32 wavefronts per CU (config 2: count 21 -> 17 us, fill 34 -> 23 us with 8 lanes; at 200 000 samples the
    // one-lane walk is ahead again, 19 / 31 us against 30 / 37 us)
    if (m * 8 <= NB_CHIP_LANES) return 8;
    if (m * 4 <= NB_CHIP_LANES) return 4;
    return 1;
}

// Any other dimension (2, 4, 5, 6): the walk of the reference, restated per lane without the shortcuts that
// three dimensions allow.  Offsets run over {-1, 0, 1} in every dimension but the last (in both when D == 2), in
// the reference's order (find_ranges_grid_ds.cu:306-338); an offset cell selects its pillar (batch, c0, c1) in the
// pillar table, and inside it the run of keys in [key - 1, key + 1] clamped to the batch
// (find_ranges_grid_ds.cu:65-165; for D == 2 the whole pillar, :203-236).  One sample per lane, ranges walked one
// after the other, hits stored one pair at a time.
template <bool FILL, bool CAPPED, int D>
__global__ void __launch_bounds__(NB_THREADS)
neighbors_generic_kernel(NbArgs a)
{
    const int lane = pccnn_lane();
    const int64_t wave = ((int64_t)blockIdx.x * NB_THREADS + threadIdx.x) >> 6;
    const int64_t base = wave * 64;
    if (base >= a.m) return;                                   // wave-uniform
    if (base + lane >= a.m) return;
    const int s = a.order ? a.order[base + lane] : (int)(base + lane);
    const int64_t at = a.presorted ? base + lane : (int64_t)s;
    const long long key0 = a.sample_keys[at];
    float sp[D], ir[D];
    int nc[D];
    long long total_cells = 1;
#pragma unroll
    for (int i = 0; i < D; ++i) {
        sp[i] = a.samples[at * D + i];
        ir[i] = __fdiv_rn(1.0f, a.radii[i]);
        nc[i] = a.num_cells[i];
        total_cells *= nc[i];
    }
    int cell0[D];
    long long aux = key0 < 0 ? 0 : key0;
#pragma unroll
    for (int i = D - 1; i >= 0; --i) { cell0[i] = (int)(aux % nc[i]); aux /= nc[i]; }
    const long long batch = aux;
    constexpr int TOP = (D - 2 > 1) ? D - 2 : 1;                 // offsets vary in dimensions 0 .. TOP
    int n_off = 3;
#pragma unroll
    for (int i = 0; i < TOP; ++i) n_off *= 3;
    constexpr int CHK = (D == 2) ? D : D - 1;                    // dimensions whose bounds are checked

    unsigned int my_off = 0;
    int raw = 0, take_step = 0, cnt = 0, err = 0;
    if (FILL) {
        my_off = s > 0 ? (unsigned int)a.ends[s - 1] : 0u;
        if (CAPPED) {
            raw = a.counts[s];
            take_step = raw < a.max_neighbors ? raw : a.max_neighbors;
        }
    }
    const unsigned int out_limit = FILL ? (unsigned int)a.t : 0u;

    for (int o = 0; o < n_off && key0 >= 0; ++o) {
        int cell[D];
        int rem = o;
        bool inside = true;
#pragma unroll
        for (int i = D - 1; i >= 0; --i) {
            int off = 0;
            if (i <= TOP) { off = rem % 3 - 1; rem /= 3; }
            if (D != 2 && i == D - 1) off = 0;
            cell[i] = cell0[i] + off;
            if (i < CHK) inside = inside && cell[i] >= 0 && cell[i] < nc[i];
        }
        if (!inside) continue;
        const long long pillar = (batch * nc[0] + cell[0]) * nc[1] + cell[1];
        if (pillar < 0 || pillar >= a.num_pillars) continue;
        int lo = a.grid_ds[2 * pillar], hi = a.grid_ds[2 * pillar + 1];
        lo = lo < 0 ? 0 : lo;
        hi = hi > a.n ? (int)a.n : hi;
        if (hi <= lo) continue;
        int first = lo, last = hi;
        if (D != 2) {
            long long key = 0, accum = 1;
#pragma unroll
            for (int i = D - 1; i >= 0; --i) { key += (long long)cell[i] * accum; accum *= nc[i]; }
            key += accum * batch;
            long long max_key = key + 1, min_key = key - 1;
            if (key / total_cells != max_key / total_cells) max_key = (key / total_cells) * total_cells + total_cells - 1;
            if (key / total_cells != min_key / total_cells) min_key = (key / total_cells) * total_cells;
            int lb = lo, ub = hi;
            while (lb < ub) {
                const int mid = lb + ((ub - lb) >> 1);
                if (a.pt_keys[mid] < min_key) lb = mid + 1; else ub = mid;
            }
            first = lb;
            lb = lo; ub = hi;
            while (lb < ub) {
                const int mid = lb + ((ub - lb) >> 1);
                if (a.pt_keys[mid] <= max_key) lb = mid + 1; else ub = mid;
            }
            last = lb;
        }
        for (int j = first; j < last; ++j) {
            // fp32, no contraction: ((s - p) * (1/r)) squared, summed over the dimensions in order from 0
            float acc = 0.0f;
#pragma unroll
            for (int i = 0; i < D; ++i) {
                const float v = (sp[i] - a.pts[(int64_t)j * D + i]) * ir[i];
                acc = acc + v * v;
            }
            if (acc < 1.0f) {
                if (FILL) {
                    bool take = true;
                    if (CAPPED) {
                        err += take_step;
                        take = err >= raw;
                        if (take) err -= raw;
                    }
                    if (take) {
                        if (my_off < out_limit)
                            ((int2 *)a.neigh)[my_off] = make_int2(a.remap ? a.remap[j] : j, s);
                        ++my_off;
                    }
                }
                ++cnt;
            }
        }
    }
    if (!FILL) a.counts[s] = cnt;
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

// Workspace layout, shared by the two calls: the pair total as int64 (written by the count call: the running
// totals in ends_out are 32-bit and wrap, this number does not) | raw counts i32[m] | scan scratch (count)
// overlaid by the packed point records float4[n] (fill).
extern "C" size_t pccnn_find_neighbors_workspace_bytes(int64_t n, int64_t m)
{
    if (m < 1) m = 1;
    if (n < 1) n = 1;
    size_t scan = pccnn_align(pccnn_scan_tmp_elems(m) * sizeof(int32_t));
    size_t rec = pccnn_align((size_t)n * sizeof(float4));
    size_t masks = pccnn_align((size_t)NB_MASK_WORDS * pccnn_ceil_div(m, 64) * 64 * sizeof(unsigned long long));
    return 256 + pccnn_align((size_t)m * sizeof(int32_t)) + masks + (scan > rec ? scan : rec) + 256;
}

static int nb_validate(const char *who, const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                       const float *samples, const int64_t *sample_keys, int64_t m, const int32_t *grid_ds,
                       int64_t num_pillars, const int32_t *cell_table, int64_t total_cells, const int32_t *num_cells, const float *radii, int d, int max_neighbors, void *workspace,
                       size_t workspace_bytes)
{
    PCCNN_REQUIRE(d >= 2 && d <= PCCNN_MAX_DIMS, PCCNN_ERR_UNSUPPORTED, "%s: d=%d is not supported (2 <= d <= 6)", who, d);
    PCCNN_REQUIRE(n >= 0 && m >= 0 && n < (1ll << 31) && m < (1ll << 31), PCCNN_ERR_INVALID, "%s: n=%lld m=%lld",
                  who, (long long)n, (long long)m);
    PCCNN_REQUIRE(max_neighbors >= 0, PCCNN_ERR_INVALID, "%s: max_neighbors=%d", who, max_neighbors);
    PCCNN_REQUIRE(num_pillars > 0, PCCNN_ERR_INVALID, "%s: num_pillars=%lld", who, (long long)num_pillars);
    PCCNN_REQUIRE(cell_table == nullptr || total_cells > 0, PCCNN_ERR_INVALID, "%s: cell_table with total_cells=%lld",
                  who, (long long)total_cells);
    PCCNN_REQUIRE(grid_ds && num_cells && radii, PCCNN_ERR_INVALID, "%s: null grid pointer", who);
    PCCNN_REQUIRE(n == 0 || (pts_sorted && pt_keys_sorted), PCCNN_ERR_INVALID, "%s: null point pointer", who);
    PCCNN_REQUIRE(m == 0 || (samples && sample_keys), PCCNN_ERR_INVALID, "%s: null sample pointer", who);
    PCCNN_REQUIRE(workspace && workspace_bytes >= pccnn_find_neighbors_workspace_bytes(n, m), PCCNN_ERR_WORKSPACE,
                  "%s: workspace of %zu bytes, need %zu", who, workspace_bytes,
                  pccnn_find_neighbors_workspace_bytes(n, m));
    return PCCNN_OK;
}

static thread_local int64_t *g_pair_total_destination = nullptr;
void pccnn_redirect_pair_total(int64_t *destination) { g_pair_total_destination = destination; }

extern "C" int pccnn_find_neighbors_count(const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                                          const float *samples, const int64_t *sample_keys, int64_t m,
                                          const int32_t *sample_order, int samples_presorted,
                                          const int32_t *grid_ds, int64_t num_pillars, const int32_t *cell_table,
                                          int64_t total_cells, const int32_t *num_cells, const float *radii, int d,
                                          int max_neighbors, int32_t *ends_out, void *workspace,
                                          size_t workspace_bytes, void *stream)
{
    int rc = nb_validate("pccnn_find_neighbors_count", pts_sorted, pt_keys_sorted, n, samples, sample_keys, m, grid_ds,
                         num_pillars, cell_table, total_cells, num_cells, radii, d, max_neighbors, workspace,
                         workspace_bytes);
    if (rc != PCCNN_OK) return rc;
    if (m == 0) return PCCNN_OK;
    PCCNN_REQUIRE(ends_out, PCCNN_ERR_INVALID, "pccnn_find_neighbors_count: null ends_out");
    hipStream_t s = (hipStream_t)stream;
    PccnnArena arena(workspace, workspace_bytes);
    int64_t *total64 = arena.take<int64_t>(1);
    if (g_pair_total_destination != nullptr) total64 = g_pair_total_destination;
    int32_t *counts = arena.take<int32_t>((size_t)m);
    const int64_t m_pad = pccnn_ceil_div(m, 64) * 64;
    unsigned long long *masks = arena.take<unsigned long long>((size_t)NB_MASK_WORDS * m_pad);
    int32_t *scan_tmp = arena.take<int32_t>(pccnn_scan_tmp_elems(m));
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_find_neighbors_count: workspace too small");
    NbArgs a;
    a.pts = pts_sorted; a.pt_keys = pt_keys_sorted; a.n = n;
    a.samples = samples; a.sample_keys = sample_keys; a.m = m;
    a.order = sample_order; a.presorted = (sample_order != nullptr && samples_presorted != 0);
    a.grid_ds = grid_ds; a.num_pillars = num_pillars;
    a.cell_table = cell_table; a.total_cells = total_cells;
    a.num_cells = num_cells; a.radii = radii; a.max_neighbors = max_neighbors;
    a.counts = counts; a.ends = nullptr; a.remap = nullptr; a.t = 0; a.neigh = nullptr; a.rec = nullptr;
    const int group = nb_group_size(n, m, d);
    // the uncapped one-lane walk leaves its decisions for the fill call
    a.masks = (group == 1 && d == 3 && max_neighbors == 0) ? masks : nullptr;
    a.m_pad = m_pad;
    int64_t waves = pccnn_ceil_div(m * group, 64);
    {
        PccnnTimed timed(PCCNN_T_NB_COUNT, s);
        const unsigned blocks = (unsigned)pccnn_ceil_div(waves, NB_THREADS / 64);
        if (group == 64) neighbors_group_kernel<false, false, 64><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
        else if (group == 16) neighbors_group_kernel<false, false, 16><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
        else if (group == 8) neighbors_group_kernel<false, false, 8><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
        else if (group == 4) neighbors_group_kernel<false, false, 4><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
        else switch (d) {
        case 3:
            if (n < (1ll << 28)) neighbors_kernel<false, false, NB_UNROLL_COUNT, true><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            else neighbors_kernel<false, false, NB_UNROLL_COUNT><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            break;
        case 2: neighbors_generic_kernel<false, false, 2><<<blocks, NB_THREADS, 0, s>>>(a); break;
        case 4: neighbors_generic_kernel<false, false, 4><<<blocks, NB_THREADS, 0, s>>>(a); break;
        case 5: neighbors_generic_kernel<false, false, 5><<<blocks, NB_THREADS, 0, s>>>(a); break;
        default: neighbors_generic_kernel<false, false, 6><<<blocks, NB_THREADS, 0, s>>>(a); break;
        }
    }
    PCCNN_LAUNCH_CHECK();
    PccnnTimed timed(PCCNN_T_SCAN, s);
    return pccnn_scan_inclusive_i32(counts, ends_out, m, max_neighbors, scan_tmp, s, total64);
}

extern "C" int pccnn_find_neighbors_fill(const float *pts_sorted, const int64_t *pt_keys_sorted, int64_t n,
                                         const float *samples, const int64_t *sample_keys, int64_t m,
                                         const int32_t *sample_order, int samples_presorted,
                                         const int32_t *grid_ds, int64_t num_pillars, const int32_t *cell_table,
                                         int64_t total_cells, const int32_t *num_cells, const float *radii, int d,
                                         int max_neighbors, const int32_t *ends, const int32_t *point_remap, int64_t t,
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
    (void)arena.take<int64_t>(1);                              // the count call's pair total
    int32_t *counts = arena.take<int32_t>((size_t)m);
    const int64_t m_pad = pccnn_ceil_div(m, 64) * 64;
    unsigned long long *masks = arena.take<unsigned long long>((size_t)NB_MASK_WORDS * m_pad);
    float4 *rec = arena.take<float4>((size_t)(n > 0 ? n : 1));
    PCCNN_REQUIRE(arena.ok(), PCCNN_ERR_WORKSPACE, "pccnn_find_neighbors_fill: workspace too small");
    NbArgs a;
    a.pts = pts_sorted; a.pt_keys = pt_keys_sorted; a.n = n;
    a.samples = samples; a.sample_keys = sample_keys; a.m = m;
    a.order = sample_order; a.presorted = (sample_order != nullptr && samples_presorted != 0);
    a.grid_ds = grid_ds; a.num_pillars = num_pillars;
    a.cell_table = cell_table; a.total_cells = total_cells;
    a.num_cells = num_cells; a.radii = radii; a.max_neighbors = max_neighbors;
    a.counts = counts; a.ends = ends; a.remap = point_remap; a.t = t; a.neigh = neigh_out; a.rec = rec;
    a.masks = masks; a.m_pad = m_pad;
    const int group = nb_group_size(n, m, d);
    int64_t waves = pccnn_ceil_div(m * group, 64);
    {
        PccnnTimed timed(PCCNN_T_NB_FILL, s);
        const unsigned blocks = (unsigned)pccnn_ceil_div(waves, NB_THREADS / 64);
        if (d == 3 && group == 1 && max_neighbors == 0) {
            // the count call left the outcome of every candidate test in the workspace: nothing is tested again
            neighbors_fill_masks_kernel<<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
        } else if (d == 3) {
            // the packed (x, y, z, id) records pay for their launch from a few ten thousand pairs on; the grouped walk
            // of a small search reads the coordinate array and the id table instead
            const bool packed = group == 1 || t >= NB_PACK_FROM_PAIRS;
            if (!packed) a.rec = nullptr;
            if (n > 0 && packed)
                pack_points_kernel<<<(unsigned)pccnn_ceil_div(n, 256), 256, 0, s>>>(pts_sorted, point_remap, n, rec);
            if (group == 64) {
                if (max_neighbors > 0) neighbors_group_kernel<true, true, 64><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
                else neighbors_group_kernel<true, false, 64><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            } else if (group == 16) {
                if (max_neighbors > 0) neighbors_group_kernel<true, true, 16><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
                else neighbors_group_kernel<true, false, 16><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            } else if (group == 8) {
                if (max_neighbors > 0) neighbors_group_kernel<true, true, 8><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
                else neighbors_group_kernel<true, false, 8><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            } else if (group == 4) {
                if (max_neighbors > 0) neighbors_group_kernel<true, true, 4><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
                else neighbors_group_kernel<true, false, 4><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            } else if (max_neighbors > 0) neighbors_kernel<true, true, NB_UNROLL_FILL><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
            else neighbors_kernel<true, false, NB_UNROLL_FILL><<<pccnn_xcd_grid(blocks, NB_XCD_CHUNK), NB_THREADS, 0, s>>>(a);
        } else {
#define NB_GENERIC(D)                                                                            \
    do {                                                                                         \
        if (max_neighbors > 0) neighbors_generic_kernel<true, true, D><<<blocks, NB_THREADS, 0, s>>>(a); \
        else neighbors_generic_kernel<true, false, D><<<blocks, NB_THREADS, 0, s>>>(a);           \
    } while (0)
            switch (d) {
            case 2: NB_GENERIC(2); break;
            case 4: NB_GENERIC(4); break;
            case 5: NB_GENERIC(5); break;
            default: NB_GENERIC(6); break;
            }
#undef NB_GENERIC
        }
    }
    PCCNN_LAUNCH_CHECK();
    return PCCNN_OK;
}
