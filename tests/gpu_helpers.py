"""Shared pieces of the GPU parity tests: run the HIP path through pccnn_lib_ops and the oracle on
the same inputs."""
import numpy as np
import torch

DEV = "cuda:0"


def t(a, dtype=None):
    out = torch.as_tensor(np.ascontiguousarray(a), device=DEV)
    return out if dtype is None else out.to(dtype)


def gpu_neighborhood(ops, pts, ids, samples, sample_ids, radius, batch_size, max_neighbors=0, use_order=True,
                     use_table=False):
    """keys -> sort -> grid -> find_neighbors through the op module; returns host arrays keyed like
    oracle.neighborhood()."""
    tp, ti = t(pts), t(ids)
    ts, tsi = t(samples), t(sample_ids)
    radii = torch.full((pts.shape[1],), float(radius), dtype=torch.float32, device=DEV) if np.isscalar(radius) \
        else t(radius)
    mn, mx = ops.bounding_box(tp, ti, batch_size)
    nc = torch.max(((mx - mn) / radii).to(torch.int32) + 1, dim=0)[0].contiguous()
    keys = ops.compute_keys(tp, ti, mn, nc, radii)
    bits = ops.key_bits_for(nc.tolist(), batch_size)
    skeys, perm, spts = ops.sort_keys(keys, bits, tp)
    ds = ops.build_grid_ds(skeys, nc, [batch_size] + nc.tolist()[0:2] + [2])
    skey = ops.compute_keys(ts, tsi, mn, nc, radii)
    order = ops.sort_keys(skey, bits)[1] if use_order else None
    table = ops.build_cell_table(skeys, batch_size * int(np.prod(nc.tolist()))) if use_table else None
    neigh_sorted, ends = ops.find_neighbors_ex(spts, skeys, ts, skey, ds, nc, radii, max_neighbors, order,
                                               cell_table=table)
    neigh, ends2 = ops.find_neighbors_ex(spts, skeys, ts, skey, ds, nc, radii, max_neighbors, order, perm,
                                         cell_table=table)
    torch.cuda.synchronize()
    assert torch.equal(ends, ends2)
    c = lambda x: x.cpu().numpy()
    return dict(aabb_min=c(mn), aabb_max=c(mx), num_cells=c(nc), keys=c(keys), perm=c(perm), sorted_keys=c(skeys),
                sorted_pts=c(spts), grid_ds=c(ds), sample_keys=c(skey), neigh_sorted=c(neigh_sorted),
                neighbors=c(neigh), ends=c(ends), radii=c(radii),
                dev=dict(pts=tp, ids=ti, samples=ts, neigh=neigh, ends=ends, radii=radii, skeys=skeys, spts=spts,
                         nc=nc, ds=ds, perm=perm))


def relerr(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def mixed_close(a, b, rtol=1e-3, atol_frac=1e-5):
    """Element-wise check beside the norm-wise relerr(): every entry within rtol of its own magnitude plus
    atol_frac of the tensor's largest magnitude (the floor that fp32 sums of terms of that size leave), so an entry a
    hundred times smaller than the largest one must still be right to about a percent of itself, not merely small."""
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return bool(np.all(np.abs(a - b) <= rtol * np.abs(b) + atol_frac * max(np.abs(b).max(), 1e-30)))
