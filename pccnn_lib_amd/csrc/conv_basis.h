// What the convolution kernels share: the basis families, the geometry argument block and the per-lane evaluation
// of one basis value.
#ifndef PCCNN_CONV_BASIS_H
#define PCCNN_CONV_BASIS_H

#include "common.h"

// Basis families (values = PCCNN_BASIS_* of the C header).
//   KP     clamp(1 - |kp_k - d| / sigma, 0, 1)                      (KPConv)
//   MLP    leaky_relu(d . A_k + b_k, 0.2) / pdf                     (MCConv)
//   KPN    the KP value / pdf                                       (KPConvN)
//   GAUSS  exp(-|kp_k - d|^2 / (2 sigma^2)) / pdf                   (PCCNN)
//   EXPLICIT  values given per pair in a [T, K] tensor              (PointConv)
//   SPH    one-hot spherical bin of d, bin 0 = the centre           (SPHConv)
//   LINEAR d . A_k + b_k                                            (PointConv's own basis op)
enum { BASIS_KP = 0, BASIS_MLP = 1, BASIS_KPN = 2, BASIS_GAUSS = 3, BASIS_EXPLICIT = 4, BASIS_SPH = 5,
       BASIS_LINEAR = 6 };

template <int BASIS> struct BasisTraits {
    static constexpr bool kernel_pts = BASIS == BASIS_KP || BASIS == BASIS_KPN || BASIS == BASIS_GAUSS;
    static constexpr bool axis = BASIS == BASIS_MLP || BASIS == BASIS_LINEAR;
    static constexpr bool uses_pdf = BASIS == BASIS_MLP || BASIS == BASIS_KPN || BASIS == BASIS_GAUSS;
    static constexpr bool pdf_grad = BASIS == BASIS_MLP || BASIS == BASIS_GAUSS;
    static constexpr bool differentiable = kernel_pts || axis;       // has a basis_bwd stage
};

struct ConvGeom {
    const float *pts;       // [n,3]
    const float *samples;   // [m,3]
    const int2 *neigh;      // [t] (point, sample)
    const int32_t *ends;    // [m]
    const float *radii;     // [3]
    const float *pdf;       // [n] or null
    const float *basis_a;   // kernel points [K,3] | axis [3,K] | explicit basis [T,K] | radial bin edges
    const float *basis_b;   // bias [K] | azimuth bin edges
    float sigma;
    int64_t n, m, t;
    int c_in, k;
    const float *basis_c;   // polar bin edges
    int nb0, nb1, nb2;      // spherical bin counts
    // Backward pass without float atomics: the feature-gradient row of a pair is stored at the pair's index (and
    // summed per point afterwards), and every sample writes a basis-parameter partial row of its own.
    int deterministic;
};

// First bin whose upper edge is >= v, the last bin when there is none.
__device__ __forceinline__ int sph_bin(float v, const float *__restrict__ edges, int count)
{
    int id = -1;
    for (int i = 0; i < count; ++i)
        if (v <= edges[i] && id < 0) id = i;
    return id < 0 ? count - 1 : id;
}

template <int BASIS> struct LaneBasis {
    float c0, c1, c2, c3;
    int kk;
    bool active;
    __device__ __forceinline__ void load(const ConvGeom &g, int k)
    {
        active = k < g.k;
        kk = k;
        c0 = c1 = c2 = c3 = 0.0f;
        if (active) {
            if (BasisTraits<BASIS>::kernel_pts) {
                c0 = g.basis_a[k * 3 + 0]; c1 = g.basis_a[k * 3 + 1]; c2 = g.basis_a[k * 3 + 2];
            } else if (BasisTraits<BASIS>::axis) {
                c0 = g.basis_a[k]; c1 = g.basis_a[g.k + k]; c2 = g.basis_a[2 * g.k + k]; c3 = g.basis_b[k];
            }
        }
    }
    // Basis value of this lane's k for a pair with normalised offset (dx,dy,dz).
    __device__ __forceinline__ float eval(const ConvGeom &g, float dx, float dy, float dz, float pdf) const
    {
        float w = 0.0f;
        if (BASIS == BASIS_KP || BASIS == BASIS_KPN) {
            const float vx = c0 - dx, vy = c1 - dy, vz = c2 - dz;
            const float d2 = fmaxf(vx * vx + vy * vy + vz * vz, 0.0f);
            const float r = 1.0f - sqrtf(d2) / g.sigma;
            w = fminf(fmaxf(r, 0.0f), 1.0f);
            if (BASIS == BASIS_KPN) w = w / pdf;
        } else if (BASIS == BASIS_GAUSS) {
            const float vx = c0 - dx, vy = c1 - dy, vz = c2 - dz;
            const float d2 = vx * vx + vy * vy + vz * vz;
            w = expf(-(d2 / (2.0f * g.sigma * g.sigma))) / pdf;
        } else if (BASIS == BASIS_MLP) {
            float a = dx * c0 + dy * c1 + dz * c2 + c3;
            a = a > 0.0f ? a : a * 0.2f;
            w = a / pdf;
        } else if (BASIS == BASIS_LINEAR) {
            w = dx * c0 + dy * c1 + dz * c2 + c3;
        } else if (BASIS == BASIS_SPH) {
            const float dist = sqrtf(dx * dx + dy * dy + dz * dz);
            const float azimuth = atanf(dy / (dx + 1e-6f));
            const float polar = acosf(fminf(fmaxf(dz / (dist + 1e-6f), -0.99999f), 0.99999f));
            int id = sph_bin(dist, g.basis_a, g.nb0) * g.nb1 * g.nb2 + sph_bin(azimuth, g.basis_b, g.nb1) * g.nb2 +
                     sph_bin(polar, g.basis_c, g.nb2) + 1;
            if (dist < 1e-4f) id = 0;
            w = (id == kk) ? 1.0f : 0.0f;
        }
        return active ? w : 0.0f;
    }
};

// Basis value for pair `pair` (global pair index) of the chunk: evaluated, or read when given explicitly.
template <int BASIS>
__device__ __forceinline__ float pair_basis(const ConvGeom &g, const LaneBasis<BASIS> &lb, int64_t pair, float dx,
                                            float dy, float dz, float pdf)
{
    if (BASIS == BASIS_EXPLICIT) return lb.active ? g.basis_a[pair * g.k + lb.kk] : 0.0f;
    return lb.eval(g, dx, dy, dz, pdf);
}

// The forward convolution that keeps the projection on chip (conv_fused.hip).
bool pccnn_conv_fused_eligible(int basis, int c_in, int k, int num_mlps, int c_out);
size_t pccnn_conv_fused_workspace_bytes(int c_in, int k, int c_out);
template <int BASIS>
int pccnn_conv_fused_forward(const ConvGeom &g, const float *feats, const float *weights, int c_out, float *out,
                             void *workspace, bool divide_by_count, bool bf16, hipStream_t s);

#endif
