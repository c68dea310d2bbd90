// pccnn_lib_ops as a compiled PyTorch extension: the module the reference builds from setup.py:7-31 and fills in
// pccnn_lib_ops/ops_list.cpp:26-54 (26 functions taking torch.Tensor arguments), bound here to the C ABI of
// libpccnn_hip.so.  Host code only: every function validates its tensors (TORCH_CHECK -> RuntimeError), allocates
// the outputs and a workspace with at::empty on the inputs' device, takes torch's current HIP stream and forwards
// raw pointers.  Positional signatures and return conventions are the reference's; the trailing keyword arguments
// (return_proj, proj, grad_mask, mirror, contraction) are this build's additions and default to the reference's
// behaviour.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <string>
#include <vector>

#include "pccnn_hip.h"

namespace {

using at::Tensor;
using OptTensor = c10::optional<Tensor>;

constexpr int kMinDims = 2, kMaxDims = 6;
constexpr int64_t kCellTableMaxCells = 1ll << 26;

void *cur_stream() { return (void *)c10::hip::getCurrentHIPStream().stream(); }

void rc_check(int rc, const char *what)
{
    if (rc != 0) {
        const char *msg = pccnn_last_error();
        TORCH_CHECK(false, what, " failed (", rc, "): ", msg ? msg : "?");
    }
}

// A GPU tensor of exactly this dtype and rank, contiguous, on `dev` (or, for the first tensor of a call, on the
// current device: the kernels are queued on that device's current stream).
const Tensor &chk(const Tensor &t, const std::string &name, at::ScalarType dtype, int ndim, const Tensor *first = nullptr)
{
    TORCH_CHECK(t.defined(), name, ": expected a torch.Tensor");
    TORCH_CHECK(t.is_cuda(), name, ": expected a GPU tensor, got device ", t.device());
    TORCH_CHECK(t.scalar_type() == dtype, name, ": expected dtype ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(ndim < 0 || t.dim() == ndim, name, ": expected ", ndim, " dimensions, got shape ", t.sizes());
    TORCH_CHECK(t.is_contiguous(), name, ": expected a contiguous tensor");
    if (first) {
        TORCH_CHECK(t.device() == first->device(), name, ": on ", t.device(), " but other arguments are on ",
                    first->device());
    } else {
        TORCH_CHECK(t.device().index() == c10::hip::current_device(), name, ": on ", t.device(),
                    ", but the current device is cuda:", (int)c10::hip::current_device(),
                    "; run the call under `with torch.cuda.device(tensor.device):`");
    }
    return t;
}

Tensor workspace(size_t bytes, const Tensor &like)
{
    return at::empty({(int64_t)std::max<size_t>(bytes, 256)}, like.options().dtype(at::kByte));
}

int dims_of(const Tensor &pts, const std::string &name, bool only_3d = false)
{
    const int d = (int)pts.size(1);
    TORCH_CHECK(d >= kMinDims && d <= kMaxDims && (!only_3d || d == 3), name, ": ", d,
                "-dimensional points are not supported (", only_3d ? "3 only" : "2 to 6 dimensions", ")");
    return d;
}

const float *fptr(const Tensor &t) { return t.data_ptr<float>(); }
const int32_t *iptr(const Tensor &t) { return t.data_ptr<int32_t>(); }
float *ofptr(const OptTensor &t) { return t.has_value() ? t->data_ptr<float>() : nullptr; }
py::object opt(const OptTensor &t) { return t.has_value() ? py::cast(*t) : py::none(); }

int key_bits_for(const std::vector<int64_t> &cells, int64_t batch)
{
    unsigned long long total = (unsigned long long)std::max<int64_t>(batch, 1);
    for (int64_t c : cells) total *= (unsigned long long)std::max<int64_t>(c, 1);
    unsigned long long v = total > 0 ? total - 1 : 0;
    int bits = 0;
    while (v) { ++bits; v >>= 1; }
    return std::max(bits, 1);
}

// Planar clouds run through the 3-D kernels with a zero third coordinate (positions, samples and kernel points
// get a zero column, axis matrices a zero row, the radii a 1): every added term is an exact zero.
bool planar(const Tensor &pts) { return pts.defined() && pts.dim() == 2 && pts.size(1) == 2; }
Tensor pad_cols(const Tensor &x, double value = 0.0) { return at::constant_pad_nd(x, {0, 1}, value).contiguous(); }
Tensor pad_rows(const Tensor &x) { return at::constant_pad_nd(x, {0, 0, 0, 1}, 0.0).contiguous(); }
OptTensor cut(const OptTensor &x)
{
    if (!x.has_value()) return x;
    return x->slice(1, 0, 2).contiguous();
}

bool is_bf16(const std::string &name, const std::string &contraction)
{
    TORCH_CHECK(contraction == "f32" || contraction == "bf16", name,
                ": contraction must be one of ('f32', 'bf16'), got '", contraction, "'");
    return contraction == "bf16";
}

// ------------------------------------------------------------------ index / grid ops

// compute_keys (pccnn_lib_ops/compute_keys/compute_keys.cuh:26-31)
Tensor compute_keys(const Tensor &pts, const Tensor &batch_ids, const Tensor &aabb_min, const Tensor &grid_size,
                    const Tensor &cell_size)
{
    chk(pts, "compute_keys: pts", at::kFloat, 2);
    chk(batch_ids, "compute_keys: batch_ids", at::kInt, 1, &pts);
    chk(aabb_min, "compute_keys: aabb_min", at::kFloat, 2, &pts);
    chk(grid_size, "compute_keys: grid_size", at::kInt, 1, &pts);
    chk(cell_size, "compute_keys: cell_size", at::kFloat, 1, &pts);
    const int d = dims_of(pts, "compute_keys");
    TORCH_CHECK(batch_ids.size(0) == pts.size(0) && aabb_min.size(1) == d && grid_size.size(0) == d &&
                    cell_size.size(0) == d,
                "compute_keys: inconsistent shapes");
    Tensor keys = at::empty({pts.size(0)}, pts.options().dtype(at::kLong));
    rc_check(pccnn_compute_keys(fptr(pts), iptr(batch_ids), fptr(aabb_min), iptr(grid_size), fptr(cell_size),
                                pts.size(0), d, keys.data_ptr<int64_t>(), cur_stream()),
             "pccnn_compute_keys");
    return keys;
}

// build_grid_ds (pccnn_lib_ops/build_grid/build_grid_ds.cuh:25-28)
Tensor build_grid_ds(const Tensor &keys, const Tensor &grid_size, const std::vector<int64_t> &out_shape)
{
    chk(keys, "build_grid_ds: keys", at::kLong, 1);
    chk(grid_size, "build_grid_ds: grid_size", at::kInt, 1, &keys);
    const int d = (int)grid_size.size(0);
    TORCH_CHECK(d >= kMinDims && d <= kMaxDims, "build_grid_ds: ", d,
                "-dimensional grids are not supported (2 to 6 dimensions)");
    bool ok = out_shape.size() == 4 && out_shape[3] == 2;
    for (int64_t v : out_shape) ok = ok && v >= 1;
    TORCH_CHECK(ok, "build_grid_ds: out_shape must be [batch, cells0, cells1, 2], got ", out_shape);
    Tensor ds = at::empty(out_shape, keys.options().dtype(at::kInt));
    rc_check(pccnn_build_grid_ds(keys.data_ptr<int64_t>(), keys.size(0), iptr(grid_size), d,
                                 out_shape[0] * out_shape[1] * out_shape[2], ds.data_ptr<int32_t>(), cur_stream()),
             "pccnn_build_grid_ds");
    return ds;
}

// find_neighbors (pccnn_lib_ops/find_neighbors/find_neighbors.cuh:33-41): count pass, the one host read-back of the
// pair total (64-bit, from the head of the workspace), fill pass.  Large searches walk the samples in cell order.
std::vector<Tensor> find_neighbors(const Tensor &pts, const Tensor &pt_keys, const Tensor &samples_in,
                                   const Tensor &sample_keys_in, const Tensor &grid_ds, const Tensor &grid_size,
                                   const Tensor &radii, int64_t max_neighbors)
{
    const std::string name = "find_neighbors";
    chk(pts, name + ": pts", at::kFloat, 2);
    chk(pt_keys, name + ": pt_keys", at::kLong, 1, &pts);
    chk(samples_in, name + ": samples", at::kFloat, 2, &pts);
    chk(sample_keys_in, name + ": sample_keys", at::kLong, 1, &pts);
    chk(grid_ds, name + ": grid_ds", at::kInt, 4, &pts);
    chk(grid_size, name + ": grid_size", at::kInt, 1, &pts);
    chk(radii, name + ": radii", at::kFloat, 1, &pts);
    const int d = dims_of(pts, name);
    const int64_t n = pts.size(0), m = samples_in.size(0);
    TORCH_CHECK(pt_keys.size(0) == n && sample_keys_in.size(0) == m && samples_in.size(1) == d &&
                    grid_size.size(0) == d && radii.size(0) == d && grid_ds.size(3) == 2,
                name, ": inconsistent shapes");
    TORCH_CHECK(max_neighbors >= 0 && max_neighbors <= INT32_MAX, name, ": max_neighbors must be >= 0");
    Tensor ends = at::empty({m}, pts.options().dtype(at::kInt));
    if (m == 0) return {at::empty({0, 2}, pts.options().dtype(at::kInt)), ends};
    const int64_t pillars = grid_ds.size(0) * grid_ds.size(1) * grid_ds.size(2);
    void *stream = cur_stream();

    Tensor samples = samples_in, sample_keys = sample_keys_in, order, table;
    int presorted = 0;
    int64_t total_cells = 0;
    if (m > 4096) {
        // queries are walked in cell order so that a wavefront's 64 queries share their cell walk
        Tensor cells_host = grid_size.cpu();
        std::vector<int64_t> cells(cells_host.data_ptr<int32_t>(), cells_host.data_ptr<int32_t>() + d);
        const int bits = key_bits_for(cells, grid_ds.size(0));
        Tensor skeys = at::empty_like(sample_keys_in), spts = at::empty_like(samples_in);
        order = at::empty({m}, pts.options().dtype(at::kInt));
        Tensor ws = workspace(pccnn_sort_keys_workspace_bytes(m), pts);
        rc_check(pccnn_sort_keys(sample_keys_in.data_ptr<int64_t>(), m, bits, skeys.data_ptr<int64_t>(),
                                 order.data_ptr<int32_t>(), fptr(samples_in), d, spts.data_ptr<float>(),
                                 ws.data_ptr(), (size_t)ws.numel(), stream),
                 "pccnn_sort_keys");
        samples = spts;
        sample_keys = skeys;
        presorted = 1;
        if (d == 3) {               // the per-cell start table belongs to the 3-dimensional walk only
            int64_t total = grid_ds.size(0) * cells[0] * cells[1] * cells[2];
            if (total <= kCellTableMaxCells) {
                table = at::empty({total + 1}, pts.options().dtype(at::kInt));
                rc_check(pccnn_build_cell_table(pt_keys.data_ptr<int64_t>(), n, total, table.data_ptr<int32_t>(), stream),
                         "pccnn_build_cell_table");
                total_cells = total;
            }
        }
    }
    const int32_t *order_p = order.defined() ? iptr(order) : nullptr;
    const int32_t *table_p = table.defined() ? iptr(table) : nullptr;
    Tensor ws = workspace(pccnn_find_neighbors_workspace_bytes(n, m), pts);
    rc_check(pccnn_find_neighbors_count(fptr(pts), pt_keys.data_ptr<int64_t>(), n, fptr(samples),
                                        sample_keys.data_ptr<int64_t>(), m, order_p, presorted, iptr(grid_ds), pillars,
                                        table_p, total_cells, iptr(grid_size), fptr(radii), d, (int)max_neighbors,
                                        ends.data_ptr<int32_t>(), ws.data_ptr(), (size_t)ws.numel(), stream),
             "pccnn_find_neighbors_count");
    // the one host read-back, as in the reference (store_neighbors.cu:257); the 64-bit total rather than ends[-1],
    // which is 32-bit and wraps
    const int64_t total = ws.slice(0, 0, 8).view(at::kLong).item<int64_t>();
    TORCH_CHECK(total >= 0 && total <= 0x7fffffffll, name,
                ": more than 2^31 - 1 pairs; the pair offsets are 32-bit as in the reference, use a smaller radius, a "
                "neighbor cap or fewer samples per call");
    Tensor neigh = at::empty({total, 2}, pts.options().dtype(at::kInt));
    rc_check(pccnn_find_neighbors_fill(fptr(pts), pt_keys.data_ptr<int64_t>(), n, fptr(samples),
                                       sample_keys.data_ptr<int64_t>(), m, order_p, presorted, iptr(grid_ds), pillars,
                                       table_p, total_cells, iptr(grid_size), fptr(radii), d, (int)max_neighbors,
                                       iptr(ends), nullptr, total, neigh.data_ptr<int32_t>(), ws.data_ptr(),
                                       (size_t)ws.numel(), stream),
             "pccnn_find_neighbors_fill");
    return {neigh, ends};
}

int pdf_args(const std::string &name, const Tensor &bandwidth, const Tensor &pts, const Tensor &neigh, const Tensor &ends)
{
    chk(pts, name + ": pts", at::kFloat, 2);
    chk(bandwidth, name + ": bandwidth", at::kFloat, 1, &pts);
    chk(neigh, name + ": neighbors", at::kInt, 2, &pts);
    chk(ends, name + ": start_ids", at::kInt, 1, &pts);
    const int d = dims_of(pts, name);
    TORCH_CHECK(bandwidth.size(0) == d && neigh.size(1) == 2 && ends.size(0) == pts.size(0), name,
                ": inconsistent shapes (the samples of a pdf are the points themselves)");
    return d;
}

// compute_pdf (pccnn_lib_ops/compute_pdf/compute_pdf.cuh:28-33)
Tensor compute_pdf(int64_t manifold_dims, const Tensor &bandwidth, const Tensor &pts, const Tensor &neigh,
                   const Tensor &ends)
{
    const int d = pdf_args("compute_pdf", bandwidth, pts, neigh, ends);
    Tensor out = at::empty({pts.size(0)}, pts.options());
    rc_check(pccnn_compute_pdf((int)manifold_dims, fptr(bandwidth), fptr(pts), pts.size(0), d, iptr(neigh),
                               neigh.size(0), iptr(ends), out.data_ptr<float>(), cur_stream()),
             "pccnn_compute_pdf");
    return out;
}

// compute_pdf_grads (pccnn_lib_ops/compute_pdf/compute_pdf.cuh:45-51)
Tensor compute_pdf_grads(int64_t manifold_dims, const Tensor &bandwidth, const Tensor &pts, const Tensor &neigh,
                         const Tensor &ends, const Tensor &in_grads_in)
{
    const int d = pdf_args("compute_pdf_grads", bandwidth, pts, neigh, ends);
    Tensor in_grads = in_grads_in.contiguous();
    chk(in_grads, "compute_pdf_grads: in_grads", at::kFloat, 1, &pts);
    TORCH_CHECK(in_grads.size(0) == pts.size(0), "compute_pdf_grads: in_grads has the wrong length");
    Tensor out = at::empty_like(pts);
    rc_check(pccnn_compute_pdf_grads((int)manifold_dims, fptr(bandwidth), fptr(pts), pts.size(0), d, iptr(neigh),
                                     neigh.size(0), iptr(ends), fptr(in_grads), out.data_ptr<float>(), cur_stream()),
             "pccnn_compute_pdf_grads");
    return out;
}

// poisson_disk_sampling (pccnn_lib_ops/poisson_disk_sampling/poisson_disk_sampling.cuh:28-32)
Tensor poisson_disk_sampling(const Tensor &sorted_keys, const Tensor &neigh, const Tensor &ends, const Tensor &grid_size)
{
    const std::string name = "poisson_disk_sampling";
    chk(sorted_keys, name + ": keys", at::kLong, 1);
    chk(neigh, name + ": neighbors", at::kInt, 2, &sorted_keys);
    chk(ends, name + ": start_ids", at::kInt, 1, &sorted_keys);
    chk(grid_size, name + ": grid_size", at::kInt, 1, &sorted_keys);
    const int64_t n = sorted_keys.size(0);
    const int d = (int)grid_size.size(0);
    TORCH_CHECK(ends.size(0) == n && d >= kMinDims && d <= kMaxDims && neigh.size(1) == 2, name, ": inconsistent shapes");
    if (n == 0) return at::empty({0, 1}, sorted_keys.options());
    Tensor sel = at::empty({n}, sorted_keys.options().dtype(at::kInt)), scan = at::empty_like(sel);
    Tensor ws = workspace(pccnn_poisson_disk_workspace_bytes(n), sorted_keys);
    void *stream = cur_stream();
    rc_check(pccnn_poisson_disk_select(sorted_keys.data_ptr<int64_t>(), n, iptr(neigh), neigh.size(0), iptr(ends),
                                       iptr(grid_size), d, sel.data_ptr<int32_t>(), scan.data_ptr<int32_t>(),
                                       ws.data_ptr(), (size_t)ws.numel(), stream),
             "pccnn_poisson_disk_select");
    const int64_t count = scan[n - 1].item<int32_t>();
    Tensor ids = at::empty({count, 1}, sorted_keys.options());
    rc_check(pccnn_compact_selected(iptr(sel), iptr(scan), n, ids.data_ptr<int64_t>(), stream), "pccnn_compact_selected");
    return ids;
}

// ------------------------------------------------------------------------ convolutions

struct ConvShape {
    int d;
    int64_t n, m, t;
    int c_in;
};

ConvShape conv_args(const std::string &name, const Tensor &pts, const Tensor &feats, const Tensor &samples,
                    const Tensor &neigh, const Tensor &ends, const Tensor &radii, bool only_3d = false)
{
    chk(pts, name + ": pts", at::kFloat, 2);
    chk(feats, name + ": features", at::kFloat, 2, &pts);
    chk(samples, name + ": samples", at::kFloat, 2, &pts);
    chk(neigh, name + ": neighbors", at::kInt, 2, &pts);
    chk(ends, name + ": start_ids", at::kInt, 1, &pts);
    chk(radii, name + ": radii", at::kFloat, 1, &pts);
    const int d = dims_of(pts, name, only_3d);
    TORCH_CHECK(feats.size(0) == pts.size(0) && samples.size(1) == d && ends.size(0) == samples.size(0) &&
                    neigh.size(1) == 2 && radii.size(0) == d,
                name, ": inconsistent shapes");
    return {d, pts.size(0), samples.size(0), neigh.size(0), (int)feats.size(1)};
}

const void *proj_arg(const std::string &name, const OptTensor &proj, int64_t m, int c_in, int k, const Tensor &like,
                     bool bf16)
{
    if (!proj.has_value()) return nullptr;
    chk(*proj, name + ": proj", bf16 ? at::kBFloat16 : at::kFloat, 3, &like);
    TORCH_CHECK(proj->size(0) == m && proj->size(1) == c_in && proj->size(2) == k, name, ": proj must be [M, Cin, K]");
    return proj->data_ptr();
}

const int32_t *mirror_arg(const std::string &name, const OptTensor &mirror, const Tensor &neigh, int64_t n, int64_t m)
{
    if (!mirror.has_value()) return nullptr;
    chk(*mirror, name + ": mirror", at::kInt, 1, &neigh);
    TORCH_CHECK(mirror->size(0) == neigh.size(0) && n == m, name, ": mirror must be [T] and needs samples == points");
    return iptr(*mirror);
}

pccnn_basis make_basis(int kind, int k, const Tensor *a, const Tensor *b, const Tensor *c, double sigma, const Tensor *pdf)
{
    pccnn_basis desc{};
    desc.kind = kind;
    desc.k = k;
    desc.sigma = (float)sigma;
    desc.a = a ? fptr(*a) : nullptr;
    desc.b = b ? fptr(*b) : nullptr;
    desc.c = c ? fptr(*c) : nullptr;
    desc.pdf = pdf ? fptr(*pdf) : nullptr;
    if (kind == PCCNN_BASIS_SPH) {
        desc.nb0 = (int)a->size(0);
        desc.nb1 = (int)b->size(0);
        desc.nb2 = (int)c->size(0);
    }
    return desc;
}

struct Generic {            // one descriptor-driven convolution: geometry optional (a caller-given basis has none)
    pccnn_basis desc;
    int k;
    const Tensor *pts, *samples, *radii;    // null for EXPLICIT
    const Tensor &feats, &neigh, &ends;
    int divide_by_count;
    int dims() const { return pts ? (int)pts->size(1) : 3; }
};

py::object out_and_proj(const Tensor &out, const Tensor &proj, bool return_proj)
{
    if (return_proj) return py::make_tuple(out, proj);
    return py::cast(out);
}

py::object generic_forward(const std::string &name, const Generic &g, const Tensor &weights, int num_mlps, int64_t c_out,
                           bool return_proj, bool bf16)
{
    const int64_t n = g.feats.size(0), m = g.ends.size(0), t = g.neigh.size(0);
    const int c_in = (int)g.feats.size(1);
    Tensor out = at::empty({m, c_out}, g.feats.options());
    // a call that does not hand the projection back lets the library build it in the workspace - or keep it on chip
    Tensor proj;
    if (return_proj) proj = at::empty({m, c_in, g.k}, g.feats.options().dtype(bf16 ? at::kBFloat16 : at::kFloat));
    Tensor ws;
    void *ws_p = nullptr;
    size_t ws_n = 0;
    if (bf16 || !return_proj || (g.pts && g.pts->size(1) != 3)) {
        ws = workspace(pccnn_conv_workspace_bytes(m, t, c_in, g.k, (int)c_out, 0), g.feats);
        ws_p = ws.data_ptr();
        ws_n = (size_t)ws.numel();
    }
    const float *pts = g.pts ? fptr(*g.pts) : nullptr, *smp = g.samples ? fptr(*g.samples) : nullptr,
                *rad = g.radii ? fptr(*g.radii) : nullptr;
    if (bf16)
        rc_check(pccnn_conv_forward_bf16(&g.desc, pts, fptr(g.feats), smp, iptr(g.neigh), iptr(g.ends), rad,
                                         fptr(weights), n, m, t, g.dims(), c_in, num_mlps, (int)c_out,
                                         g.divide_by_count, out.data_ptr<float>(),
                                         return_proj ? (uint16_t *)proj.data_ptr() : nullptr, ws_p, ws_n, cur_stream()),
                 "pccnn_conv_forward_bf16");
    else
        rc_check(pccnn_conv_forward(&g.desc, pts, fptr(g.feats), smp, iptr(g.neigh), iptr(g.ends), rad, fptr(weights), n,
                                    m, t, g.dims(), c_in, num_mlps, (int)c_out, g.divide_by_count,
                                    out.data_ptr<float>(), return_proj ? proj.data_ptr<float>() : nullptr, ws_p, ws_n,
                                    cur_stream()),
                 "pccnn_conv_forward");
    return out_and_proj(out, proj, return_proj);
}

struct Grads {
    OptTensor d_w, d_f, d_a, d_b, d_pdf, d_p, d_s;
};

void generic_backward(const std::string &name, const Generic &g, const Tensor &weights, int num_mlps, int64_t c_out,
                      const Tensor &in_grads_in, const OptTensor &proj, const OptTensor &mirror, int grad_mask, bool bf16,
                      Grads &out)
{
    const int64_t n = g.feats.size(0), m = g.ends.size(0), t = g.neigh.size(0);
    const int c_in = (int)g.feats.size(1);
    Tensor in_grads = in_grads_in.contiguous();
    chk(in_grads, name + ": in_grads", at::kFloat, 2, &g.feats);
    TORCH_CHECK(in_grads.size(0) == m && in_grads.size(1) == c_out, name, ": in_grads must be [M, Cout]");
    const void *proj_p = proj_arg(name, proj, m, c_in, g.k, g.feats, bf16);
    const int32_t *mirror_p = g.pts ? mirror_arg(name, mirror, g.neigh, n, m) : nullptr;
    // the larger workspace when the pass without atomics is asked for, and when the library may take the per-pair
    // rows by itself (a mirror index, wide rows, no basis / position / density gradients)
    const bool rows_route = mirror_p != nullptr && c_in > 32 && (grad_mask & PCCNN_GRAD_FEATS) &&
                            !(grad_mask & (PCCNN_GRAD_BASIS_PARAMS | PCCNN_GRAD_PDF | PCCNN_GRAD_PTS));
    Tensor ws = workspace(((grad_mask & PCCNN_GRAD_DETERMINISTIC) || rows_route)
                              ? pccnn_conv_workspace_bytes_deterministic(n, m, t, c_in, g.k, (int)c_out)
                              : pccnn_conv_workspace_bytes(m, t, c_in, g.k, (int)c_out, 1),
                          g.feats);
    const float *pts = g.pts ? fptr(*g.pts) : nullptr, *smp = g.samples ? fptr(*g.samples) : nullptr,
                *rad = g.radii ? fptr(*g.radii) : nullptr;
    if (bf16)
        rc_check(pccnn_conv_backward_bf16(&g.desc, pts, fptr(g.feats), smp, iptr(g.neigh), iptr(g.ends), rad,
                                          fptr(weights), fptr(in_grads), (const uint16_t *)proj_p, mirror_p, grad_mask,
                                          n, m, t, g.dims(), c_in, num_mlps, (int)c_out, g.divide_by_count,
                                          ofptr(out.d_w), ofptr(out.d_f), ofptr(out.d_a), ofptr(out.d_b),
                                          ofptr(out.d_pdf), ofptr(out.d_p), ofptr(out.d_s), ws.data_ptr(),
                                          (size_t)ws.numel(), cur_stream()),
                 "pccnn_conv_backward_bf16");
    else
        rc_check(pccnn_conv_backward(&g.desc, pts, fptr(g.feats), smp, iptr(g.neigh), iptr(g.ends), rad, fptr(weights),
                                     fptr(in_grads), (const float *)proj_p, mirror_p, grad_mask, n, m, t, g.dims(), c_in,
                                     num_mlps, (int)c_out, g.divide_by_count, ofptr(out.d_w), ofptr(out.d_f),
                                     ofptr(out.d_a), ofptr(out.d_b), ofptr(out.d_pdf), ofptr(out.d_p), ofptr(out.d_s),
                                     ws.data_ptr(), (size_t)ws.numel(), cur_stream()),
                 "pccnn_conv_backward");
}

Tensor generic_weight_var(const Generic &g)
{
    const int64_t n = g.feats.size(0), m = g.ends.size(0), t = g.neigh.size(0);
    const int c_in = (int)g.feats.size(1);
    Tensor out = at::empty({1}, g.feats.options());
    Tensor ws = workspace(pccnn_conv_weight_var_workspace_bytes(m, t, c_in, g.k), g.feats);
    rc_check(pccnn_conv_weight_var(&g.desc, g.pts ? fptr(*g.pts) : nullptr, fptr(g.feats),
                                   g.samples ? fptr(*g.samples) : nullptr, iptr(g.neigh), iptr(g.ends),
                                   g.radii ? fptr(*g.radii) : nullptr, n, m, t, g.dims(), c_in, g.divide_by_count,
                                   out.data_ptr<float>(), ws.data_ptr(), (size_t)ws.numel(), cur_stream()),
             "pccnn_conv_weight_var");
    return out.reshape({});
}

OptTensor like_if(const Tensor &like, int mask, int bit) { return (mask & bit) ? OptTensor(at::empty_like(like)) : OptTensor(); }

// ---- the kernel-point families: KPConv (kpconv.cuh:32-90), KPConvN (kpconvn.cuh:32-93), PCCNN (pccnn.cuh:32-93)

int kp_family_args(const std::string &name, int kind, const Tensor &pts, const OptTensor &pdf, const Tensor &feats,
                   const Tensor &samples, const Tensor &neigh, const Tensor &ends, const Tensor &radii,
                   const Tensor &kernel_pts)
{
    ConvShape s = conv_args(name, pts, feats, samples, neigh, ends, radii);
    chk(kernel_pts, name + ": kernel_pts", at::kFloat, 2, &pts);
    if (kind != PCCNN_BASIS_KP) {
        chk(*pdf, name + ": pdf", at::kFloat, 1, &pts);
        TORCH_CHECK(pdf->size(0) == s.n && kernel_pts.size(1) == s.d, name, ": pdf must be [N] and kernel_pts [K, D]");
    } else {
        TORCH_CHECK(kernel_pts.size(1) == s.d, name, ": weights must be [K*Cin, Cout] and kernel_pts [K, D]");
    }
    return (int)kernel_pts.size(0);
}

py::object kp_family_forward(const std::string &name, int kind, const Tensor &pts, const OptTensor &pdf,
                             const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
                             const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights,
                             bool return_proj, const std::string &contraction)
{
    if (planar(pts))
        return kp_family_forward(name, kind, pad_cols(pts), pdf, feats, pad_cols(samples), neigh, ends,
                                 pad_cols(radii, 1.0), pad_cols(kernel_pts), sigma, weights, return_proj, contraction);
    const bool bf16 = is_bf16(name, contraction);
    TORCH_CHECK(!bf16 || kind == PCCNN_BASIS_KP, name, ": the bf16 contraction is offered for kp_conv and mc_conv");
    const int k = kp_family_args(name, kind, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts);
    chk(weights, name + ": weights", at::kFloat, 2, &pts);
    TORCH_CHECK(weights.size(0) == (int64_t)k * feats.size(1), name, ": weights must be [K*Cin, Cout]");
    Generic g{make_basis(kind, k, &kernel_pts, nullptr, nullptr, sigma, pdf.has_value() ? &*pdf : nullptr), k, &pts,
              &samples, &radii, feats, neigh, ends, 0};
    return generic_forward(name, g, weights, 1, weights.size(1), return_proj, bf16);
}

// -> [dW, dFeat, dKernelPts, (dPdf for PCCNN,) dPts, dSamples]
py::list kp_family_backward(const std::string &name, int kind, const Tensor &pts, const OptTensor &pdf,
                            const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
                            const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights,
                            const Tensor &in_grads, const OptTensor &proj, int64_t grad_mask, const OptTensor &mirror,
                            const std::string &contraction)
{
    if (planar(pts)) {
        py::list g = kp_family_backward(name, kind, pad_cols(pts), pdf, feats, pad_cols(samples), neigh, ends,
                                        pad_cols(radii, 1.0), pad_cols(kernel_pts), sigma, weights, in_grads, proj,
                                        grad_mask, mirror, contraction);
        const size_t last = g.size();
        for (size_t i : {(size_t)2, last - 2, last - 1})
            if (!g[i].is_none()) g[i] = py::cast(g[i].cast<Tensor>().slice(1, 0, 2).contiguous());
        return g;
    }
    const bool bf16 = is_bf16(name, contraction);
    TORCH_CHECK(!bf16 || kind == PCCNN_BASIS_KP, name, ": the bf16 contraction is offered for kp_conv and mc_conv");
    const int k = kp_family_args(name, kind, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts);
    chk(weights, name + ": weights", at::kFloat, 2, &pts);
    TORCH_CHECK(weights.size(0) == (int64_t)k * feats.size(1), name, ": inconsistent shapes");
    const int mask = (int)grad_mask;
    Grads gr;
    gr.d_w = like_if(weights, mask, PCCNN_GRAD_WEIGHTS);
    gr.d_f = like_if(feats, mask, PCCNN_GRAD_FEATS);
    gr.d_a = like_if(kernel_pts, mask, PCCNN_GRAD_BASIS_PARAMS);
    if (kind == PCCNN_BASIS_GAUSS) gr.d_pdf = like_if(*pdf, mask, PCCNN_GRAD_PDF);
    gr.d_p = like_if(pts, mask, PCCNN_GRAD_PTS);
    gr.d_s = like_if(samples, mask, PCCNN_GRAD_PTS);
    Generic g{make_basis(kind, k, &kernel_pts, nullptr, nullptr, sigma, pdf.has_value() ? &*pdf : nullptr), k, &pts,
              &samples, &radii, feats, neigh, ends, 0};
    generic_backward(name, g, weights, 1, weights.size(1), in_grads, proj, mirror, mask, bf16, gr);
    py::list out;
    out.append(opt(gr.d_w));
    out.append(opt(gr.d_f));
    out.append(opt(gr.d_a));
    if (kind == PCCNN_BASIS_GAUSS) out.append(opt(gr.d_pdf));
    out.append(opt(gr.d_p));
    out.append(opt(gr.d_s));
    return out;
}

Tensor kp_family_weight_var(const std::string &name, int kind, const Tensor &pts, const OptTensor &pdf,
                            const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
                            const Tensor &radii, const Tensor &kernel_pts, double sigma)
{
    if (planar(pts))
        return kp_family_weight_var(name, kind, pad_cols(pts), pdf, feats, pad_cols(samples), neigh, ends,
                                    pad_cols(radii, 1.0), pad_cols(kernel_pts), sigma);
    const int k = kp_family_args(name, kind, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts);
    Generic g{make_basis(kind, k, &kernel_pts, nullptr, nullptr, sigma, pdf.has_value() ? &*pdf : nullptr), k, &pts,
              &samples, &radii, feats, neigh, ends, 0};
    return generic_weight_var(g);
}

// ---- MCConv (pccnn_lib_ops/pcconvs/mcconv.cuh:32-92)

struct McShape {
    int k, num_mlps;
    int64_t c_out;
};

McShape mc_args(const std::string &name, const ConvShape &s, const Tensor &pts, const Tensor &pdf, const Tensor &axis,
                const Tensor &bias, const Tensor *weights)
{
    chk(pdf, name + ": pdf", at::kFloat, 1, &pts);
    chk(axis, name + ": axis", at::kFloat, 2, &pts);
    chk(bias, name + ": bias", at::kFloat, 2, &pts);
    const int k = (int)axis.size(1);
    TORCH_CHECK(pdf.size(0) == s.n && axis.size(0) == s.d && bias.size(0) == 1 && bias.size(1) == k, name,
                ": axis must be [D, H*mlps], bias [1, H*mlps], pdf [N]");
    if (!weights) return {k, 1, 0};
    chk(*weights, name + ": weights", at::kFloat, 3, &pts);
    const int num_mlps = (int)weights->size(0);
    TORCH_CHECK(weights->size(1) * num_mlps == (int64_t)k * s.c_in, name,
                ": axis must be [D, H*mlps], bias [1, H*mlps], weights [mlps, H*Cin, Cout/mlps]");
    return {k, num_mlps, weights->size(0) * weights->size(2)};
}

py::object mc_conv(const Tensor &pts, const Tensor &pdf, const Tensor &feats, const Tensor &samples, const Tensor &neigh,
                   const Tensor &ends, const Tensor &radii, const Tensor &axis, const Tensor &bias, const Tensor &weights,
                   bool return_proj, const std::string &contraction)
{
    const std::string name = "mc_conv";
    if (planar(pts))
        return mc_conv(pad_cols(pts), pdf, feats, pad_cols(samples), neigh, ends, pad_cols(radii, 1.0), pad_rows(axis),
                       bias, weights, return_proj, contraction);
    const bool bf16 = is_bf16(name, contraction);
    ConvShape s = conv_args(name, pts, feats, samples, neigh, ends, radii);
    McShape mc = mc_args(name, s, pts, pdf, axis, bias, &weights);
    Generic g{make_basis(PCCNN_BASIS_MLP, mc.k, &axis, &bias, nullptr, 1.0, &pdf), mc.k, &pts, &samples, &radii, feats,
              neigh, ends, 0};
    return generic_forward(name, g, weights, mc.num_mlps, mc.c_out, return_proj, bf16);
}

py::list mc_conv_grads(const Tensor &pts, const Tensor &pdf, const Tensor &feats, const Tensor &samples,
                       const Tensor &neigh, const Tensor &ends, const Tensor &radii, const Tensor &axis,
                       const Tensor &bias, const Tensor &weights, const Tensor &in_grads, const OptTensor &proj,
                       int64_t grad_mask, const OptTensor &mirror, const std::string &contraction)
{
    const std::string name = "mc_conv_grads";
    if (planar(pts)) {
        py::list g = mc_conv_grads(pad_cols(pts), pdf, feats, pad_cols(samples), neigh, ends, pad_cols(radii, 1.0),
                                   pad_rows(axis), bias, weights, in_grads, proj, grad_mask, mirror, contraction);
        if (!g[2].is_none()) g[2] = py::cast(g[2].cast<Tensor>().slice(0, 0, 2).contiguous());
        for (size_t i : {(size_t)5, (size_t)6})
            if (!g[i].is_none()) g[i] = py::cast(g[i].cast<Tensor>().slice(1, 0, 2).contiguous());
        return g;
    }
    const bool bf16 = is_bf16(name, contraction);
    ConvShape s = conv_args(name, pts, feats, samples, neigh, ends, radii);
    McShape mc = mc_args(name, s, pts, pdf, axis, bias, &weights);
    const int mask = (int)grad_mask;
    Grads gr;
    gr.d_w = like_if(weights, mask, PCCNN_GRAD_WEIGHTS);
    gr.d_f = like_if(feats, mask, PCCNN_GRAD_FEATS);
    gr.d_a = like_if(axis, mask, PCCNN_GRAD_BASIS_PARAMS);
    gr.d_b = like_if(bias, mask, PCCNN_GRAD_BASIS_PARAMS);
    gr.d_pdf = like_if(pdf, mask, PCCNN_GRAD_PDF);
    gr.d_p = like_if(pts, mask, PCCNN_GRAD_PTS);
    gr.d_s = like_if(samples, mask, PCCNN_GRAD_PTS);
    Generic g{make_basis(PCCNN_BASIS_MLP, mc.k, &axis, &bias, nullptr, 1.0, &pdf), mc.k, &pts, &samples, &radii, feats,
              neigh, ends, 0};
    generic_backward(name, g, weights, mc.num_mlps, mc.c_out, in_grads, proj, mirror, mask, bf16, gr);
    py::list out;
    for (const OptTensor *t : {&gr.d_w, &gr.d_f, &gr.d_a, &gr.d_b, &gr.d_pdf, &gr.d_p, &gr.d_s}) out.append(opt(*t));
    return out;
}

Tensor mc_conv_weight_var(const Tensor &pts, const Tensor &pdf, const Tensor &feats, const Tensor &samples,
                          const Tensor &neigh, const Tensor &ends, const Tensor &radii, const Tensor &axis,
                          const Tensor &bias)
{
    const std::string name = "mc_conv_weight_var";
    if (planar(pts))
        return mc_conv_weight_var(pad_cols(pts), pdf, feats, pad_cols(samples), neigh, ends, pad_cols(radii, 1.0),
                                  pad_rows(axis), bias);
    ConvShape s = conv_args(name, pts, feats, samples, neigh, ends, radii);
    McShape mc = mc_args(name, s, pts, pdf, axis, bias, nullptr);
    Generic g{make_basis(PCCNN_BASIS_MLP, mc.k, &axis, &bias, nullptr, 1.0, &pdf), mc.k, &pts, &samples, &radii, feats,
              neigh, ends, 0};
    return generic_weight_var(g);
}

// ---- SPHConv (pccnn_lib_ops/pcconvs/sphconv.cuh:19-55)

Generic sph_args(const std::string &name, const Tensor &pts, const Tensor &feats, const Tensor &samples,
                 const Tensor &neigh, const Tensor &ends, const Tensor &radii, const Tensor &radial, const Tensor &azimuth,
                 const Tensor &polar)
{
    conv_args(name, pts, feats, samples, neigh, ends, radii, true);          // spherical coordinates: 3-D only
    const Tensor *bins[3] = {&radial, &azimuth, &polar};
    const char *what[3] = {"radial", "azimuth", "polar"};
    for (int i = 0; i < 3; ++i) {
        chk(*bins[i], name + ": " + what[i] + " bins", at::kFloat, 1, &pts);
        TORCH_CHECK(bins[i]->size(0) >= 1, name, ": empty ", what[i], " bins");
    }
    const int k = (int)(radial.size(0) * azimuth.size(0) * polar.size(0) + 1);
    return Generic{make_basis(PCCNN_BASIS_SPH, k, &radial, &azimuth, &polar, 1.0, nullptr), k, &pts, &samples, &radii,
                   feats, neigh, ends, 1};
}

py::object sph_conv(const Tensor &pts, const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
                    const Tensor &radii, const Tensor &radial, const Tensor &azimuth, const Tensor &polar,
                    const Tensor &weights, bool return_proj)
{
    Generic g = sph_args("sph_conv", pts, feats, samples, neigh, ends, radii, radial, azimuth, polar);
    chk(weights, "sph_conv: weights", at::kFloat, 2, &pts);
    TORCH_CHECK(weights.size(0) == (int64_t)g.k * feats.size(1), "sph_conv: weights must be [K*Cin, Cout]");
    return generic_forward("sph_conv", g, weights, 1, weights.size(1), return_proj, false);
}

py::list sph_conv_grads(const Tensor &pts, const Tensor &feats, const Tensor &samples, const Tensor &neigh,
                        const Tensor &ends, const Tensor &radii, const Tensor &radial, const Tensor &azimuth,
                        const Tensor &polar, const Tensor &weights, const Tensor &in_grads, const OptTensor &proj,
                        int64_t grad_mask)
{
    Generic g = sph_args("sph_conv_grads", pts, feats, samples, neigh, ends, radii, radial, azimuth, polar);
    chk(weights, "sph_conv_grads: weights", at::kFloat, 2, &pts);
    TORCH_CHECK(weights.size(0) == (int64_t)g.k * feats.size(1), "sph_conv_grads: inconsistent shapes");
    const int mask = (int)grad_mask & (PCCNN_GRAD_WEIGHTS | PCCNN_GRAD_FEATS | PCCNN_GRAD_DETERMINISTIC);
    Grads gr;
    gr.d_w = like_if(weights, mask, PCCNN_GRAD_WEIGHTS);
    gr.d_f = like_if(feats, mask, PCCNN_GRAD_FEATS);
    generic_backward("sph_conv_grads", g, weights, 1, weights.size(1), in_grads, proj, OptTensor(), mask, false, gr);
    py::list out;
    out.append(opt(gr.d_w));
    out.append(opt(gr.d_f));
    return out;
}

Tensor sph_conv_weight_var(const Tensor &pts, const Tensor &feats, const Tensor &samples, const Tensor &neigh,
                           const Tensor &ends, const Tensor &radii, const Tensor &radial, const Tensor &azimuth,
                           const Tensor &polar)
{
    return generic_weight_var(sph_args("sph_conv_weight_var", pts, feats, samples, neigh, ends, radii, radial, azimuth,
                                       polar));
}

// ---- PointConv (pccnn_lib_ops/pcconvs/pointconv.cuh:20-56)

struct LinearShape {
    int d, k;
};

LinearShape linear_basis_args(const std::string &name, const Tensor &pts, const Tensor &radii, const Tensor &samples,
                              const Tensor &neigh, const Tensor &axis, const Tensor &bias)
{
    chk(pts, name + ": pts", at::kFloat, 2);
    const int d = dims_of(pts, name);
    chk(samples, name + ": samples", at::kFloat, 2, &pts);
    chk(neigh, name + ": neighbors", at::kInt, 2, &pts);
    chk(radii, name + ": radii", at::kFloat, 1, &pts);
    chk(axis, name + ": axis", at::kFloat, 2, &pts);
    chk(bias, name + ": bias", at::kFloat, -1, &pts);
    const int k = (int)axis.size(1);
    TORCH_CHECK(samples.size(1) == d && neigh.size(1) == 2 && radii.size(0) == d && axis.size(0) == d && bias.numel() == k,
                name, ": axis must be [D, K], bias [1, K] or [K], radii [D]");
    return {d, k};
}

Tensor point_conv_basis(const Tensor &pts, const Tensor &radii, const Tensor &samples, const Tensor &neigh,
                        const Tensor &axis, const Tensor &bias)
{
    const std::string name = "point_conv_basis";
    if (planar(pts))
        return point_conv_basis(pad_cols(pts), pad_cols(radii, 1.0), pad_cols(samples), neigh, pad_rows(axis), bias);
    LinearShape s = linear_basis_args(name, pts, radii, samples, neigh, axis, bias);
    const int64_t t = neigh.size(0);
    Tensor out = at::empty({t, s.k}, pts.options());
    rc_check(pccnn_linear_basis_forward(fptr(pts), fptr(samples), iptr(neigh), fptr(radii), fptr(axis), fptr(bias),
                                        pts.size(0), samples.size(0), t, s.d, s.k, out.data_ptr<float>(), cur_stream()),
             "pccnn_linear_basis_forward");
    return out;
}

std::vector<Tensor> point_conv_basis_grads(const Tensor &pts, const Tensor &radii, const Tensor &samples,
                                           const Tensor &neigh, const Tensor &axis, const Tensor &bias,
                                           const Tensor &in_grads_in)
{
    const std::string name = "point_conv_basis_grads";
    if (planar(pts)) {
        std::vector<Tensor> g = point_conv_basis_grads(pad_cols(pts), pad_cols(radii, 1.0), pad_cols(samples), neigh,
                                                       pad_rows(axis), bias, in_grads_in);
        return {g[0].slice(1, 0, 2).contiguous(), g[1].slice(1, 0, 2).contiguous(), g[2].slice(0, 0, 2).contiguous(),
                g[3]};
    }
    LinearShape s = linear_basis_args(name, pts, radii, samples, neigh, axis, bias);
    const int64_t t = neigh.size(0);
    Tensor in_grads = in_grads_in.contiguous();
    chk(in_grads, name + ": in_grads", at::kFloat, 2, &pts);
    TORCH_CHECK(in_grads.size(0) == t && in_grads.size(1) == s.k, name, ": in_grads must be [T, K]");
    Tensor d_p = at::empty_like(pts), d_s = at::empty_like(samples), d_a = at::empty_like(axis);
    Tensor d_b = at::empty({1, s.k}, pts.options());
    Tensor ws = workspace(pccnn_linear_basis_workspace_bytes(t), pts);
    rc_check(pccnn_linear_basis_backward(fptr(pts), fptr(samples), iptr(neigh), fptr(radii), fptr(axis), fptr(bias),
                                         fptr(in_grads), pts.size(0), samples.size(0), t, s.d, s.k,
                                         d_p.data_ptr<float>(), d_s.data_ptr<float>(), d_a.data_ptr<float>(),
                                         d_b.data_ptr<float>(), ws.data_ptr(), (size_t)ws.numel(), cur_stream()),
             "pccnn_linear_basis_backward");
    return {d_p, d_s, d_a, d_b};
}

Generic explicit_args(const std::string &name, const Tensor &basis, const Tensor &feats, const Tensor &neigh,
                      const Tensor &ends)
{
    chk(basis, name + ": basis", at::kFloat, 2);
    chk(feats, name + ": features", at::kFloat, 2, &basis);
    chk(neigh, name + ": neighbors", at::kInt, 2, &basis);
    chk(ends, name + ": start_ids", at::kInt, 1, &basis);
    TORCH_CHECK(basis.size(0) == neigh.size(0) && neigh.size(1) == 2, name,
                ": basis must be [T, K] and neighbors [T, 2]");
    const int k = (int)basis.size(1);
    return Generic{make_basis(PCCNN_BASIS_EXPLICIT, k, &basis, nullptr, nullptr, 1.0, nullptr), k, nullptr, nullptr,
                   nullptr, feats, neigh, ends, 0};
}

py::object point_conv(const Tensor &basis, const Tensor &feats, const Tensor &neigh, const Tensor &ends,
                      const Tensor &weights, bool return_proj)
{
    Generic g = explicit_args("point_conv", basis, feats, neigh, ends);
    chk(weights, "point_conv: weights", at::kFloat, 2, &basis);
    TORCH_CHECK(weights.size(0) == (int64_t)g.k * feats.size(1), "point_conv: weights must be [K*Cin, Cout]");
    return generic_forward("point_conv", g, weights, 1, weights.size(1), return_proj, false);
}

py::list point_conv_grads(const Tensor &basis, const Tensor &feats, const Tensor &neigh, const Tensor &ends,
                          const Tensor &weights, const Tensor &in_grads, const OptTensor &proj, int64_t grad_mask)
{
    Generic g = explicit_args("point_conv_grads", basis, feats, neigh, ends);
    chk(weights, "point_conv_grads: weights", at::kFloat, 2, &basis);
    TORCH_CHECK(weights.size(0) == (int64_t)g.k * feats.size(1), "point_conv_grads: inconsistent shapes");
    const int mask = (int)grad_mask & (PCCNN_GRAD_WEIGHTS | PCCNN_GRAD_FEATS | PCCNN_GRAD_BASIS_PARAMS |
                                      PCCNN_GRAD_DETERMINISTIC);
    Grads gr;
    gr.d_w = like_if(weights, mask, PCCNN_GRAD_WEIGHTS);
    gr.d_f = like_if(feats, mask, PCCNN_GRAD_FEATS);
    gr.d_a = like_if(basis, mask, PCCNN_GRAD_BASIS_PARAMS);
    generic_backward("point_conv_grads", g, weights, 1, weights.size(1), in_grads, proj, OptTensor(), mask, false, gr);
    py::list out;
    out.append(opt(gr.d_w));
    out.append(opt(gr.d_f));
    out.append(opt(gr.d_a));
    return out;
}

Tensor point_conv_weight_var(const Tensor &basis, const Tensor &feats, const Tensor &neigh, const Tensor &ends)
{
    return generic_weight_var(explicit_args("point_conv_weight_var", basis, feats, neigh, ends));
}

}  // namespace

PYBIND11_MODULE(pccnn_lib_ops, mod)
{
    namespace py = pybind11;
    using namespace pybind11::literals;
    mod.doc() = "pccnn_lib's native op module (pccnn_lib_ops/ops_list.cpp:26-54) over libpccnn_hip.so for MI355X";
    const OptTensor none;
    const int all = PCCNN_GRAD_ALL;

    // pccnn_lib_ops/ops_list.cpp:27-32
    mod.def("build_grid_ds", &build_grid_ds, "Build the pillar table of a grid");
    mod.def("compute_keys", &compute_keys, "Compute the cell keys of points");
    mod.def("find_neighbors", &find_neighbors, "Find the neighbors of samples within a radius");
    mod.def("compute_pdf", &compute_pdf, "Gaussian kernel density at every point");
    mod.def("compute_pdf_grads", &compute_pdf_grads, "Gradient of compute_pdf w.r.t. the points");
    mod.def("poisson_disk_sampling", &poisson_disk_sampling, "Poisson-disk selection");

    // ops_list.cpp:33-35
    mod.def("mc_conv", &mc_conv, "pts"_a, "pdf"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a,
            "axis"_a, "bias"_a, "weights"_a, "return_proj"_a = false, "contraction"_a = "f32");
    mod.def("mc_conv_grads", &mc_conv_grads, "pts"_a, "pdf"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a,
            "radii"_a, "axis"_a, "bias"_a, "weights"_a, "in_grads"_a, "proj"_a = none, "grad_mask"_a = all,
            "mirror"_a = none, "contraction"_a = "f32");
    mod.def("mc_conv_weight_var", &mc_conv_weight_var);

    // ops_list.cpp:36-40
    mod.def("point_conv_basis", &point_conv_basis);
    mod.def("point_conv_basis_grads", &point_conv_basis_grads);
    mod.def("point_conv", &point_conv, "basis"_a, "feats"_a, "neighbors"_a, "start_ids"_a, "weights"_a,
            "return_proj"_a = false);
    mod.def("point_conv_grads", &point_conv_grads, "basis"_a, "feats"_a, "neighbors"_a, "start_ids"_a, "weights"_a,
            "in_grads"_a, "proj"_a = none, "grad_mask"_a = all);
    mod.def("point_conv_weight_var", &point_conv_weight_var);

    // ops_list.cpp:41-43
    mod.def(
        "kp_conv",
        [](const Tensor &pts, const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
           const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights, bool return_proj,
           const std::string &contraction) {
            return kp_family_forward("kp_conv", PCCNN_BASIS_KP, pts, OptTensor(), feats, samples, neigh, ends, radii,
                                     kernel_pts, sigma, weights, return_proj, contraction);
        },
        "pts"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a, "kernel_pts"_a, "sigma"_a, "weights"_a,
        "return_proj"_a = false, "contraction"_a = "f32");
    mod.def(
        "kp_conv_grads",
        [](const Tensor &pts, const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
           const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights, const Tensor &in_grads,
           const OptTensor &proj, int64_t grad_mask, const OptTensor &mirror, const std::string &contraction) {
            return kp_family_backward("kp_conv_grads", PCCNN_BASIS_KP, pts, OptTensor(), feats, samples, neigh, ends,
                                      radii, kernel_pts, sigma, weights, in_grads, proj, grad_mask, mirror, contraction);
        },
        "pts"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a, "kernel_pts"_a, "sigma"_a, "weights"_a,
        "in_grads"_a, "proj"_a = none, "grad_mask"_a = all, "mirror"_a = none, "contraction"_a = "f32");
    mod.def("kp_conv_weight_var",
            [](const Tensor &pts, const Tensor &feats, const Tensor &samples, const Tensor &neigh, const Tensor &ends,
               const Tensor &radii, const Tensor &kernel_pts, double sigma) {
                return kp_family_weight_var("kp_conv_weight_var", PCCNN_BASIS_KP, pts, OptTensor(), feats, samples,
                                            neigh, ends, radii, kernel_pts, sigma);
            });

    // ops_list.cpp:44-46
    mod.def(
        "kp_conv_n",
        [](const Tensor &pts, const Tensor &pdf, const Tensor &feats, const Tensor &samples, const Tensor &neigh,
           const Tensor &ends, const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights,
           bool return_proj) {
            return kp_family_forward("kp_conv_n", PCCNN_BASIS_KPN, pts, pdf, feats, samples, neigh, ends, radii,
                                     kernel_pts, sigma, weights, return_proj, "f32");
        },
        "pts"_a, "pdf"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a, "kernel_pts"_a, "sigma"_a,
        "weights"_a, "return_proj"_a = false);
    mod.def(
        "kp_conv_n_grads",
        [](const Tensor &pts, const Tensor &pdf, const Tensor &feats, const Tensor &samples, const Tensor &neigh,
           const Tensor &ends, const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights,
           const Tensor &in_grads, const OptTensor &proj, int64_t grad_mask, const OptTensor &mirror) {
            return kp_family_backward("kp_conv_n_grads", PCCNN_BASIS_KPN, pts, pdf, feats, samples, neigh, ends, radii,
                                      kernel_pts, sigma, weights, in_grads, proj, grad_mask, mirror, "f32");
        },
        "pts"_a, "pdf"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a, "kernel_pts"_a, "sigma"_a,
        "weights"_a, "in_grads"_a, "proj"_a = none, "grad_mask"_a = all, "mirror"_a = none);
    mod.def("kp_conv_n_weight_var",
            [](const Tensor &pts, const Tensor &pdf, const Tensor &feats, const Tensor &samples, const Tensor &neigh,
               const Tensor &ends, const Tensor &radii, const Tensor &kernel_pts, double sigma) {
                return kp_family_weight_var("kp_conv_n_weight_var", PCCNN_BASIS_KPN, pts, pdf, feats, samples, neigh,
                                            ends, radii, kernel_pts, sigma);
            });

    // ops_list.cpp:47-49
    mod.def("sph_conv", &sph_conv, "pts"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a,
            "radial_bins"_a, "azimuth_bins"_a, "polar_bins"_a, "weights"_a, "return_proj"_a = false);
    mod.def("sph_conv_grads", &sph_conv_grads, "pts"_a, "feats"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a,
            "radial_bins"_a, "azimuth_bins"_a, "polar_bins"_a, "weights"_a, "in_grads"_a, "proj"_a = none,
            "grad_mask"_a = PCCNN_GRAD_WEIGHTS | PCCNN_GRAD_FEATS);
    mod.def("sph_conv_weight_var", &sph_conv_weight_var);

    // ops_list.cpp:50-52 (note the feats-before-pdf argument order of this family)
    mod.def(
        "pccnn",
        [](const Tensor &pts, const Tensor &feats, const Tensor &pdf, const Tensor &samples, const Tensor &neigh,
           const Tensor &ends, const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights,
           bool return_proj) {
            return kp_family_forward("pccnn", PCCNN_BASIS_GAUSS, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts,
                                     sigma, weights, return_proj, "f32");
        },
        "pts"_a, "feats"_a, "pdf"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a, "kernel_pts"_a, "sigma"_a,
        "weights"_a, "return_proj"_a = false);
    mod.def(
        "pccnn_grads",
        [](const Tensor &pts, const Tensor &feats, const Tensor &pdf, const Tensor &samples, const Tensor &neigh,
           const Tensor &ends, const Tensor &radii, const Tensor &kernel_pts, double sigma, const Tensor &weights,
           const Tensor &in_grads, const OptTensor &proj, int64_t grad_mask, const OptTensor &mirror) {
            return kp_family_backward("pccnn_grads", PCCNN_BASIS_GAUSS, pts, pdf, feats, samples, neigh, ends, radii,
                                      kernel_pts, sigma, weights, in_grads, proj, grad_mask, mirror, "f32");
        },
        "pts"_a, "feats"_a, "pdf"_a, "samples"_a, "neighbors"_a, "start_ids"_a, "radii"_a, "kernel_pts"_a, "sigma"_a,
        "weights"_a, "in_grads"_a, "proj"_a = none, "grad_mask"_a = all, "mirror"_a = none);
    mod.def("pccnn_weight_variance",
            [](const Tensor &pts, const Tensor &feats, const Tensor &pdf, const Tensor &samples, const Tensor &neigh,
               const Tensor &ends, const Tensor &radii, const Tensor &kernel_pts, double sigma) {
                return kp_family_weight_var("pccnn_weight_variance", PCCNN_BASIS_GAUSS, pts, pdf, feats, samples, neigh,
                                            ends, radii, kernel_pts, sigma);
            });

    mod.attr("GRAD_WEIGHTS") = PCCNN_GRAD_WEIGHTS;
    mod.attr("GRAD_FEATS") = PCCNN_GRAD_FEATS;
    mod.attr("GRAD_BASIS_PARAMS") = PCCNN_GRAD_BASIS_PARAMS;
    mod.attr("GRAD_PDF") = PCCNN_GRAD_PDF;
    mod.attr("GRAD_PTS") = PCCNN_GRAD_PTS;
    mod.attr("GRAD_ALL") = PCCNN_GRAD_ALL;
    mod.attr("GRAD_DETERMINISTIC") = PCCNN_GRAD_DETERMINISTIC;
    mod.attr("REFERENCE_NAMES") = py::make_tuple(
        "build_grid_ds", "compute_keys", "find_neighbors", "compute_pdf", "compute_pdf_grads", "poisson_disk_sampling",
        "mc_conv", "mc_conv_grads", "mc_conv_weight_var", "point_conv_basis", "point_conv_basis_grads", "point_conv",
        "point_conv_grads", "point_conv_weight_var", "kp_conv", "kp_conv_grads", "kp_conv_weight_var", "kp_conv_n",
        "kp_conv_n_grads", "kp_conv_n_weight_var", "sph_conv", "sph_conv_grads", "sph_conv_weight_var", "pccnn",
        "pccnn_grads", "pccnn_weight_variance");
    mod.attr("binding") = "compiled";
}
