"""Drop-in counterpart of the reference's ``pccnn_lib_ops`` extension module.

The reference exports 26 host functions taking ``torch.Tensor`` arguments
(pccnn_lib_ops/ops_list.cpp:26-54).  This module exports the same names with the same positional
signatures and return conventions; each call validates its tensors, allocates the outputs and a
workspace with torch (device memory and the current stream are all torch is used for) and
forwards raw pointers to ``libpccnn_hip.so``.  Tensors must be CUDA/HIP tensors, contiguous and of
exactly the reference's dtypes; anything else raises ``RuntimeError`` (the reference reads such
input as raw memory).

Beyond the reference's names, ``bounding_box``, ``sort_keys`` and ``find_neighbors_ex`` expose the
native replacements of the torch / torch_scatter glue the reference keeps in Python
(pccnn_lib/pc/BoundingBox.py:17-18, pccnn_lib/pc/Grid.py:52,68-70, pccnn_lib/pc/Neighborhood.py:27-53).
"""
import ctypes

import torch

from . import _lib

_P = _lib.P


# torch's current stream as a raw hipStream_t: the C-level getter when this torch has it (a fraction of a
# microsecond), else through the Stream object (several microseconds, once per native call)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    if _raw_stream is not None:
        return _P(_raw_stream(torch.cuda.current_device()))
    return _P(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return _P(t.data_ptr())


def _chk(t, name, dtype, ndim=None, device=None):
    if not isinstance(t, torch.Tensor):
        raise RuntimeError("%s: expected a torch.Tensor, got %s" % (name, type(t).__name__))
    if not t.is_cuda:
        raise RuntimeError("%s: expected a GPU tensor, got device %s" % (name, t.device))
    if t.dtype != dtype:
        raise RuntimeError("%s: expected dtype %s, got %s" % (name, dtype, t.dtype))
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError("%s: expected %d dimensions, got shape %s" % (name, ndim, tuple(t.shape)))
    if not t.is_contiguous():
        raise RuntimeError("%s: expected a contiguous tensor" % name)
    if device is not None:
        if t.device != device:
            raise RuntimeError("%s: on %s but other arguments are on %s" % (name, t.device, device))
    elif t.device.index != torch.cuda.current_device():
        # the kernels are queued on the current device's stream (see _stream): the tensors must live there
        raise RuntimeError("%s: on %s, but the current device is cuda:%d; run the call under "
                           "`with torch.cuda.device(tensor.device):`" % (name, t.device, torch.cuda.current_device()))
    return t


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


MIN_DIMS, MAX_DIMS = 2, 6


def _dims(pts, name):
    d = pts.shape[1]
    if d < MIN_DIMS or d > MAX_DIMS:
        raise RuntimeError("%s: %d-dimensional points are not supported (%d to %d dimensions)"
                           % (name, d, MIN_DIMS, MAX_DIMS))
    return d


# ------------------------------------------------------------------ index / grid ops


def bounding_box(pts, batch_ids, batch_size):
    """Per-cloud (min - 1e-6, max + 1e-6) -> (f32[B,D], f32[B,D])."""
    _chk(pts, "bounding_box: pts", torch.float32, 2)
    _chk(batch_ids, "bounding_box: batch_ids", torch.int32, 1, pts.device)
    d = _dims(pts, "bounding_box")
    batch_size = int(batch_size)
    mn = torch.empty((batch_size, d), dtype=torch.float32, device=pts.device)
    mx = torch.empty_like(mn)
    _lib.call("pccnn_bounding_box", _ptr(pts), _ptr(batch_ids), pts.shape[0], d, batch_size, _ptr(mn), _ptr(mx),
              _stream())
    return mn, mx


def bounding_box_host(pts, batch_ids, batch_size):
    """``bounding_box`` and the same box on the host, from one native call that ends with its one read-back:
    -> (f32[B,D], f32[B,D], (numpy f32[B,D], numpy f32[B,D]))."""
    import numpy as np
    _chk(pts, "bounding_box: pts", torch.float32, 2)
    _chk(batch_ids, "bounding_box: batch_ids", torch.int32, 1, pts.device)
    d = _dims(pts, "bounding_box")
    batch_size = int(batch_size)
    mn = torch.empty((batch_size, d), dtype=torch.float32, device=pts.device)
    mx = torch.empty_like(mn)
    host = np.empty((2, batch_size, d), dtype=np.float32)
    _lib.call("pccnn_bounding_box_host", _ptr(pts), _ptr(batch_ids), pts.shape[0], d, batch_size, _ptr(mn), _ptr(mx),
              _P(host.ctypes.data), _P(host.ctypes.data + host[0].nbytes), _stream())
    return mn, mx, (host[0], host[1])


# Pinned blocks that kernels write into by themselves (torch's host allocator does not know about those writes):
# the last few are kept, each with an event recorded behind its kernels, and a block is let go only after its event
# has passed, so that it cannot be handed out again while a write into it is still on its way.
_LANDINGS = []

# Reads of a polled pinned word before the host falls back to waiting for the event recorded behind the kernels
# (tests lower it to exercise that fall-back).
SPIN_LIMIT = 100000


def set_fused_forward(on):
    """``set_fused_forward(True)``: forward convolutions that do not return their projection keep it on chip when the
    shape allows it (one kernel from the gather to the output).  Off by default - the two-kernel path is the faster
    one on MI355X.  Returns the previous setting.  Process-wide."""
    return bool(_lib.load().pccnn_set_fused_forward(1 if on else 0))


def _keep_until_written(landing, done):
    _LANDINGS.append((landing, done))
    if len(_LANDINGS) > 8:
        _, oldest = _LANDINGS.pop(0)
        oldest.synchronize()


def bounding_box_host_later(pts, batch_ids, batch_size):
    """``bounding_box`` with the host copy on its way: -> (f32[B,D], f32[B,D], fetch), where ``fetch()`` returns the
    two numpy arrays once they are there.  The box kernels write them into pinned memory themselves, a flag word
    last, and ``fetch`` polls that word (with many clouds: two copies and an event).  Whatever the caller does
    before it calls ``fetch`` runs beside the device's work."""
    import numpy as np
    _chk(pts, "bounding_box: pts", torch.float32, 2)
    _chk(batch_ids, "bounding_box: batch_ids", torch.int32, 1, pts.device)
    d = _dims(pts, "bounding_box")
    batch_size = int(batch_size)
    count = batch_size * d
    box = torch.empty((2, batch_size, d), dtype=torch.float32, device=pts.device)
    base = box.data_ptr()
    landing = torch.empty((2 * count + 1,), dtype=torch.float32, pin_memory=True)
    words = landing.numpy().view(np.int32)
    words[2 * count] = -1
    polled = ctypes.c_int(0)
    _lib.call("pccnn_bounding_box_queued", _ptr(pts), _ptr(batch_ids), pts.shape[0], d, batch_size, _P(base),
              _P(base + 4 * count), _P(landing.data_ptr()), ctypes.byref(polled), _stream())
    done = torch.cuda.Event()
    done.record()
    _keep_until_written(landing, done)

    def fetch():
        spins = 0
        while polled.value and words[2 * count] < 0:
            spins += 1
            if spins > SPIN_LIMIT:
                break
        if not polled.value or words[2 * count] < 0:
            done.synchronize()
        host = landing.numpy()[:2 * count].reshape(2, batch_size, d)
        return host[0], host[1]
    fetch.polled = bool(polled.value)
    return box[0], box[1], fetch


def num_cells(aabb_min, aabb_max, cell_size):
    """Grid size i32[D] = max over the clouds of int32((max - min) / cell_size) + 1 (pccnn_lib/pc/Grid.py:26-28)."""
    name = "num_cells"
    _chk(aabb_min, name + ": aabb_min", torch.float32, 2)
    dev = aabb_min.device
    _chk(aabb_max, name + ": aabb_max", torch.float32, 2, dev)
    _chk(cell_size, name + ": cell_size", torch.float32, 1, dev)
    b, d = aabb_min.shape
    if tuple(aabb_max.shape) != (b, d) or cell_size.shape[0] != d or d < MIN_DIMS or d > MAX_DIMS or b < 1:
        raise RuntimeError(name + ": aabb_min / aabb_max must be [B, D], cell_size [D], 2 <= D <= 6")
    out = torch.empty((d,), dtype=torch.int32, device=dev)
    _lib.call("pccnn_num_cells", _ptr(aabb_min), _ptr(aabb_max), _ptr(cell_size), b, d, _ptr(out), _stream())
    return out


def compute_keys(pts, batch_ids, aabb_min, grid_size, cell_size):
    """compute_keys(pts f32[N,D], batch_ids i32[N], aabb_min f32[B,D], grid_size i32[D], cell_size f32[D]) -> i64[N]
    (pccnn_lib_ops/compute_keys/compute_keys.cuh:26-31)."""
    _chk(pts, "compute_keys: pts", torch.float32, 2)
    dev = pts.device
    _chk(batch_ids, "compute_keys: batch_ids", torch.int32, 1, dev)
    _chk(aabb_min, "compute_keys: aabb_min", torch.float32, 2, dev)
    _chk(grid_size, "compute_keys: grid_size", torch.int32, 1, dev)
    _chk(cell_size, "compute_keys: cell_size", torch.float32, 1, dev)
    d = _dims(pts, "compute_keys")
    if batch_ids.shape[0] != pts.shape[0] or aabb_min.shape[1] != d or grid_size.shape[0] != d or cell_size.shape[0] != d:
        raise RuntimeError("compute_keys: inconsistent shapes")
    keys = torch.empty((pts.shape[0],), dtype=torch.int64, device=dev)
    _lib.call("pccnn_compute_keys", _ptr(pts), _ptr(batch_ids), _ptr(aabb_min), _ptr(grid_size), _ptr(cell_size),
              pts.shape[0], d, _ptr(keys), _stream())
    return keys


def sort_keys(keys, key_bits=0, pts=None):
    """Stable radix sort of cell keys.  Returns (sorted_keys i64[N], perm i32[N], sorted_pts f32[N,D] or None)."""
    _chk(keys, "sort_keys: keys", torch.int64, 1)
    n = keys.shape[0]
    dev = keys.device
    skeys = torch.empty_like(keys)
    perm = torch.empty((n,), dtype=torch.int32, device=dev)
    spts = None
    d = 3
    if pts is not None:
        _chk(pts, "sort_keys: pts", torch.float32, 2, dev)
        d = _dims(pts, "sort_keys")
        if pts.shape[0] != n:
            raise RuntimeError("sort_keys: pts and keys differ in length")
        spts = torch.empty_like(pts)
    ws = _workspace(_lib.load().pccnn_sort_keys_workspace_bytes(n), dev)
    _lib.call("pccnn_sort_keys", _ptr(keys), n, int(key_bits), _ptr(skeys), _ptr(perm),
              _ptr(pts) if pts is not None else _P(0), d, _ptr(spts) if spts is not None else _P(0),
              _ptr(ws), ws.numel(), _stream())
    return skeys, perm, spts


def build_grid_ds(keys, grid_size, out_shape):
    """build_grid_ds(sorted keys i64[N], grid_size i32[D], out_shape [B, nc0, nc1, 2]) -> i32 tensor of out_shape
    (pccnn_lib_ops/build_grid/build_grid_ds.cuh:25-28)."""
    _chk(keys, "build_grid_ds: keys", torch.int64, 1)
    _chk(grid_size, "build_grid_ds: grid_size", torch.int32, 1, keys.device)
    out_shape = [int(v) for v in out_shape]
    d = grid_size.shape[0]
    if d < MIN_DIMS or d > MAX_DIMS:
        raise RuntimeError("build_grid_ds: %d-dimensional grids are not supported (%d to %d dimensions)"
                           % (d, MIN_DIMS, MAX_DIMS))
    if len(out_shape) != 4 or out_shape[3] != 2 or min(out_shape) < 1:
        raise RuntimeError("build_grid_ds: out_shape must be [batch, cells0, cells1, 2], got %s" % (out_shape,))
    ds = torch.empty(out_shape, dtype=torch.int32, device=keys.device)
    _lib.call("pccnn_build_grid_ds", _ptr(keys), keys.shape[0], _ptr(grid_size), d,
              out_shape[0] * out_shape[1] * out_shape[2], _ptr(ds), _stream())
    return ds


def key_bits_for(grid_size_host, batch_size):
    """Number of significant key bits for a grid of the given host-side size."""
    total = int(batch_size)
    for v in grid_size_host:
        total *= int(v)
    return max(1, (max(total, 1) - 1).bit_length())


# Largest grid (in cells) for which the per-cell start table is built: 2^26 cells = 256 MiB of int32.
CELL_TABLE_MAX_CELLS = 1 << 26


def build_cell_table(sorted_keys, total_cells):
    """i32[total_cells + 1]: index of the first sorted point with key >= c, for every cell c."""
    _chk(sorted_keys, "build_cell_table: keys", torch.int64, 1)
    table = torch.empty((int(total_cells) + 1,), dtype=torch.int32, device=sorted_keys.device)
    _lib.call("pccnn_build_cell_table", _ptr(sorted_keys), sorted_keys.shape[0], int(total_cells), _ptr(table),
              _stream())
    return table


def grid_build(pts, batch_ids, aabb_min, grid_size, cell_size, key_bits, out_shape, with_cell_table):
    """compute_keys + sort_keys + build_grid_ds (+ build_cell_table) of one grid as a single native call (what
    pccnn_lib/pc/Grid.py:40-72 does in several).  Returns (keys i64[N], sorted keys i64[N], perm i32[N], sorted
    points f32[N,D], grid_ds i32 of ``out_shape`` = [B, nc0, nc1, 2], cell table i32[cells + 1] or None)."""
    name = "grid_build"
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(batch_ids, name + ": batch_ids", torch.int32, 1, dev)
    _chk(aabb_min, name + ": aabb_min", torch.float32, 2, dev)
    _chk(grid_size, name + ": grid_size", torch.int32, 1, dev)
    _chk(cell_size, name + ": cell_size", torch.float32, 1, dev)
    d = _dims(pts, name)
    n = pts.shape[0]
    out_shape = [int(v) for v in out_shape]
    if batch_ids.shape[0] != n or aabb_min.shape[1] != d or grid_size.shape[0] != d or cell_size.shape[0] != d \
            or len(out_shape) != 4 or out_shape[3] != 2 or min(out_shape) < 1:
        raise RuntimeError(name + ": inconsistent shapes")
    keys = torch.empty((n,), dtype=torch.int64, device=dev)
    skeys = torch.empty_like(keys)
    perm = torch.empty((n,), dtype=torch.int32, device=dev)
    spts = torch.empty_like(pts)
    ds = torch.empty(out_shape, dtype=torch.int32, device=dev)
    total_cells, table = 0, None
    if with_cell_table:
        total_cells = int(with_cell_table)
        table = torch.empty((total_cells + 1,), dtype=torch.int32, device=dev)
    ws = _workspace(_lib.load().pccnn_grid_build_workspace_bytes(n), dev)
    _lib.call("pccnn_grid_build", _ptr(pts), _ptr(batch_ids), _ptr(aabb_min), _ptr(grid_size), _ptr(cell_size), n, d,
              int(key_bits), out_shape[0] * out_shape[1] * out_shape[2], total_cells, _ptr(keys), _ptr(skeys),
              _ptr(perm), _ptr(spts), _ptr(ds), _optr(table), _ptr(ws), ws.numel(), _stream())
    return keys, skeys, perm, spts, ds, table


def find_neighbors_ex(pts, pt_keys, samples, sample_keys, grid_ds, grid_size, radii, max_neighbors,
                      sample_order=None, point_remap=None, cell_table=None, samples_presorted=False):
    """find_neighbors with the native extras: ``sample_order`` (i32[M], samples listed in key order),
    ``point_remap`` (i32[N], written through to column 0 of the result), ``cell_table`` (from
    build_cell_table: replaces the per-pillar binary searches by two table reads) and ``samples_presorted``
    (``samples`` / ``sample_keys`` are given in ``sample_order`` order, as sort_keys returns them; the result
    still refers to the samples by their own indices ``sample_order[i]``)."""
    name = "find_neighbors"
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(pt_keys, name + ": pt_keys", torch.int64, 1, dev)
    _chk(samples, name + ": samples", torch.float32, 2, dev)
    _chk(sample_keys, name + ": sample_keys", torch.int64, 1, dev)
    _chk(grid_ds, name + ": grid_ds", torch.int32, 4, dev)
    _chk(grid_size, name + ": grid_size", torch.int32, 1, dev)
    _chk(radii, name + ": radii", torch.float32, 1, dev)
    d = _dims(pts, name)
    n, m = pts.shape[0], samples.shape[0]
    if pt_keys.shape[0] != n or sample_keys.shape[0] != m or samples.shape[1] != d or grid_size.shape[0] != d \
            or radii.shape[0] != d or grid_ds.shape[3] != 2:
        raise RuntimeError(name + ": inconsistent shapes")
    max_neighbors = int(max_neighbors)
    if max_neighbors < 0:
        raise RuntimeError(name + ": max_neighbors must be >= 0")
    if sample_order is not None:
        _chk(sample_order, name + ": sample_order", torch.int32, 1, dev)
        if sample_order.shape[0] != m:
            raise RuntimeError(name + ": sample_order has the wrong length")
    if point_remap is not None:
        _chk(point_remap, name + ": point_remap", torch.int32, 1, dev)
        if point_remap.shape[0] != n:
            raise RuntimeError(name + ": point_remap has the wrong length")
    pillars = grid_ds.shape[0] * grid_ds.shape[1] * grid_ds.shape[2]
    table_p, total_cells = _P(0), 0
    if cell_table is not None:
        _chk(cell_table, name + ": cell_table", torch.int32, 1, dev)
        table_p, total_cells = _ptr(cell_table), cell_table.shape[0] - 1
    ends = torch.empty((m,), dtype=torch.int32, device=dev)
    if m == 0:
        return [torch.empty((0, 2), dtype=torch.int32, device=dev), ends]
    ws = _workspace(_lib.load().pccnn_find_neighbors_workspace_bytes(n, m), dev)
    order_p = _ptr(sample_order) if sample_order is not None else _P(0)
    presorted = 1 if (samples_presorted and sample_order is not None) else 0
    _lib.call("pccnn_find_neighbors_count", _ptr(pts), _ptr(pt_keys), n, _ptr(samples), _ptr(sample_keys), m, order_p,
              presorted, _ptr(grid_ds), pillars, table_p, total_cells, _ptr(grid_size), _ptr(radii), d, max_neighbors, _ptr(ends),
              _ptr(ws), ws.numel(), _stream())
    # the one host read-back, as in the reference; the 64-bit total from the head of the workspace rather than
    # ends[-1], which is 32-bit and wraps (to a negative or, beyond 2^32 pairs, to a plausible positive number)
    total = int(ws[:8].view(torch.int64).item())
    if total < 0 or total > 0x7fffffff:
        raise RuntimeError(name + ": more than 2^31 - 1 pairs; the pair offsets are 32-bit as in the reference, "
                                  "use a smaller radius, a neighbor cap or fewer samples per call")
    neigh = torch.empty((total, 2), dtype=torch.int32, device=dev)
    _lib.call("pccnn_find_neighbors_fill", _ptr(pts), _ptr(pt_keys), n, _ptr(samples), _ptr(sample_keys), m, order_p,
              presorted, _ptr(grid_ds), pillars, table_p, total_cells, _ptr(grid_size), _ptr(radii), d, max_neighbors, _ptr(ends),
              _ptr(point_remap) if point_remap is not None else _P(0), total, _ptr(neigh), _ptr(ws), ws.numel(),
              _stream())
    return [neigh, ends]


def find_neighbors(pts, pt_keys, samples, sample_keys, grid_ds, grid_size, radii, max_neighbors):
    """find_neighbors(sorted pts, sorted keys, samples, sample keys, grid_ds, grid_size, radii, max_neighbors)
    -> [neigh i32[T,2] = (sorted point index, sample index), ends i32[M]]
    (pccnn_lib_ops/find_neighbors/find_neighbors.cuh:33-41)."""
    order, table = None, None
    if isinstance(sample_keys, torch.Tensor) and sample_keys.is_cuda and sample_keys.dim() == 1 \
            and sample_keys.shape[0] > 4096 and isinstance(grid_size, torch.Tensor) and grid_ds.dim() == 4 \
            and isinstance(pt_keys, torch.Tensor) and pt_keys.dtype == torch.int64:
        # queries are walked in cell order so that a wavefront's 64 queries share their cell walk
        cells = grid_size.tolist()
        bits = key_bits_for(cells, grid_ds.shape[0])
        skeys, order, spts = sort_keys(sample_keys, bits, samples)
        if len(cells) == 3:          # the per-cell start table belongs to the 3-dimensional walk only
            total = grid_ds.shape[0] * cells[0] * cells[1] * cells[2]
            if total <= CELL_TABLE_MAX_CELLS:
                table = build_cell_table(pt_keys, total)
        return find_neighbors_ex(pts, pt_keys, spts, skeys, grid_ds, grid_size, radii, max_neighbors, order,
                                 cell_table=table, samples_presorted=True)
    return find_neighbors_ex(pts, pt_keys, samples, sample_keys, grid_ds, grid_size, radii, max_neighbors, order,
                             cell_table=table)


def grid_build_sized(pts, batch_ids, aabb_min, num_cells_host, cell_size, batch_size):
    """``grid_build`` for a grid whose size is known on the host (a list of D ints): the device copy of that size
    is written by the same native call.  Returns (num_cells i32[D], keys, sorted keys, perm, sorted points, grid_ds
    [B, nc0, nc1, 2], cell table or None)."""
    name = "grid_build"
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(batch_ids, name + ": batch_ids", torch.int32, 1, dev)
    _chk(aabb_min, name + ": aabb_min", torch.float32, 2, dev)
    _chk(cell_size, name + ": cell_size", torch.float32, 1, dev)
    d = _dims(pts, name)
    n = pts.shape[0]
    batch_size = int(batch_size)
    cells = [int(v) for v in num_cells_host]
    if batch_ids.shape[0] != n or tuple(aabb_min.shape) != (batch_size, d) or cell_size.shape[0] != d \
            or len(cells) != d or min(cells) < 1:
        raise RuntimeError(name + ": inconsistent shapes")
    total = batch_size
    for c in cells:
        total *= c
    with_table = 1 if (d == 3 and total <= CELL_TABLE_MAX_CELLS) else 0
    num = torch.empty((d,), dtype=torch.int32, device=dev)
    keys = torch.empty((n,), dtype=torch.int64, device=dev)
    skeys = torch.empty_like(keys)
    perm = torch.empty((n,), dtype=torch.int32, device=dev)
    spts = torch.empty_like(pts)
    ds = torch.empty((batch_size, cells[0], cells[1], 2), dtype=torch.int32, device=dev)
    table = torch.empty((total + 1,), dtype=torch.int32, device=dev) if with_table else None
    ws = _workspace(_lib.load().pccnn_grid_build_workspace_bytes(n), dev)
    _lib.call("pccnn_grid_build_sized", _ptr(pts), _ptr(batch_ids), _ptr(aabb_min), (ctypes.c_int32 * d)(*cells),
              _ptr(cell_size), n, d, batch_size, key_bits_for(cells, batch_size), with_table, _ptr(num), _ptr(keys),
              _ptr(skeys), _ptr(perm), _ptr(spts), _ptr(ds), _optr(table), _ptr(ws), ws.numel(), _stream())
    return num, keys, skeys, perm, spts, ds, table


def neighborhood_build(pts, batch_ids, aabb_min, num_cells_host, cell_size, batch_size, samples, sample_batch_ids,
                       max_neighbors, remap_points):
    """A 3-D layer's neighborhood from the cloud's box: the grid over ``pts`` (as ``grid_build_sized``), the samples
    in key order, the count pass and the pair total in one native call, the pair list in a second one (what
    pccnn_lib/pc/layers/MCConv.py:136-140 with pccnn_lib/pc/Neighborhood.py:27-53 does).  ``samples`` None: the
    cloud's own points.  ``remap_points``: column 0 of the pairs holds original point indices, else indices into
    the sorted copy.  Returns (grid tuple of ``grid_build_sized``, pairs i32[T,2], ends i32[M])."""
    name = "neighborhood_build"
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(batch_ids, name + ": batch_ids", torch.int32, 1, dev)
    _chk(aabb_min, name + ": aabb_min", torch.float32, 2, dev)
    _chk(cell_size, name + ": cell_size", torch.float32, 1, dev)
    n = pts.shape[0]
    batch_size = int(batch_size)
    max_neighbors = int(max_neighbors)
    if pts.shape[1] != 3 or batch_ids.shape[0] != n or tuple(aabb_min.shape) != (batch_size, 3) \
            or cell_size.shape[0] != 3 or n < 1 or max_neighbors < 0:
        raise RuntimeError(name + ": 3-D points [N,3] (N > 0), batch_ids [N], aabb_min [B,3], cell_size [3], three "
                                  "grid sizes, max_neighbors >= 0")
    m = n
    if samples is not None:
        _chk(samples, name + ": samples", torch.float32, 2, dev)
        _chk(sample_batch_ids, name + ": sample batch_ids", torch.int32, 1, dev)
        m = samples.shape[0]
        if samples.shape[1] != 3 or sample_batch_ids.shape[0] != m or m < 1:
            raise RuntimeError(name + ": samples [M,3] (M > 0) with batch_ids [M]")
    lib = _lib.load()
    num = torch.empty((3,), dtype=torch.int32, device=dev)
    keys = torch.empty((n,), dtype=torch.int64, device=dev)
    skeys = torch.empty_like(keys)
    perm = torch.empty((n,), dtype=torch.int32, device=dev)
    spts = torch.empty_like(pts)
    ends = torch.empty((m,), dtype=torch.int32, device=dev)
    sort_ws = _workspace(lib.pccnn_grid_build_workspace_bytes(max(n, m)), dev)
    ws = _workspace(lib.pccnn_find_neighbors_workspace_bytes(n, m), dev)
    if samples is not None:
        # unsorted keys | sorted keys (i64 each) | sorted points (3 f32) | order (i32): 32 bytes per sample
        sbuf = torch.empty((4 * m,), dtype=torch.int64, device=dev)
        sb = sbuf.data_ptr()
        s_tmp, s_keys, s_pts, s_order = _P(sb), _P(sb + 8 * m), _P(sb + 16 * m), _P(sb + 28 * m)
        f_pts, f_keys, f_order = s_pts, s_keys, s_order
        samples_p, sample_ids_p = _ptr(samples), _ptr(sample_batch_ids)
    else:
        s_tmp = s_keys = s_pts = s_order = samples_p = sample_ids_p = _P(0)
        f_pts, f_keys, f_order = _ptr(spts), _ptr(skeys), _ptr(perm)
    # (the grid size last: when it is a callable it may have to wait for the cloud's box to arrive on the host)
    cells = [int(v) for v in (num_cells_host() if callable(num_cells_host) else num_cells_host)]
    if len(cells) != 3 or min(cells) < 1:
        raise RuntimeError(name + ": three positive grid sizes")
    pillars = batch_size * cells[0] * cells[1]
    total_cells = pillars * cells[2]
    with_table = 1 if total_cells <= CELL_TABLE_MAX_CELLS else 0
    ds = torch.empty((batch_size, cells[0], cells[1], 2), dtype=torch.int32, device=dev)
    table = torch.empty((total_cells + 1,), dtype=torch.int32, device=dev) if with_table else None
    bits = key_bits_for(cells, batch_size)
    total = ctypes.c_int64(0)
    _lib.call("pccnn_neighborhood_count", _ptr(pts), _ptr(batch_ids), n, batch_size, _ptr(aabb_min), _ptr(cell_size),
              (ctypes.c_int32 * 3)(*cells), bits, with_table, _ptr(num), _ptr(keys), _ptr(skeys), _ptr(perm), _ptr(spts),
              _ptr(ds), _optr(table), samples_p, sample_ids_p, m, s_tmp, s_keys, s_order, s_pts, max_neighbors,
              _ptr(ends), ctypes.byref(total), _ptr(sort_ws), sort_ws.numel(), _ptr(ws), ws.numel(), _stream())
    total = total.value
    if total < 0 or total > 0x7fffffff:
        raise RuntimeError(name + ": more than 2^31 - 1 pairs; the pair offsets are 32-bit as in the reference, "
                                  "use a smaller radius, a neighbor cap or fewer samples per call")
    neigh = torch.empty((total, 2), dtype=torch.int32, device=dev)
    _lib.call("pccnn_find_neighbors_fill", _ptr(spts), _ptr(skeys), n, f_pts, f_keys, m, f_order, 1, _ptr(ds), pillars,
              _optr(table), total_cells if with_table else 0, _ptr(num), _ptr(cell_size), 3, max_neighbors, _ptr(ends),
              _ptr(perm) if remap_points else _P(0), total, _ptr(neigh), _ptr(ws), ws.numel(), _stream())
    return (num, keys, skeys, perm, spts, ds, table), neigh, ends


# ------------------------------------------------------------------------------ pdf


def _pdf_args(name, bandwidth, pts, neigh, ends):
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(bandwidth, name + ": bandwidth", torch.float32, 1, dev)
    _chk(neigh, name + ": neighbors", torch.int32, 2, dev)
    _chk(ends, name + ": start_ids", torch.int32, 1, dev)
    d = _dims(pts, name)
    if bandwidth.shape[0] != d or neigh.shape[1] != 2 or ends.shape[0] != pts.shape[0]:
        raise RuntimeError(name + ": inconsistent shapes (the samples of a pdf are the points themselves)")
    return d


def compute_pdf(manifold_dims, bandwidth, pts, neigh, ends):
    """compute_pdf(manifold_dims, bandwidth f32[D], pts, neighbors, start_ids) -> f32[N]
    (pccnn_lib_ops/compute_pdf/compute_pdf.cuh:28-33).

    Every pair gathers its neighbor's coordinates by original index, as in the reference.  On a large cloud whose
    points sit in memory in no spatial order that is a cache line per pair (a million scattered points with 19
    neighbors each: 1.85 GB fetched for 170 MB of pairs and points, 241 us); compute_pdf_sorted on the grid's
    sorted copy, or compute_pdf_grid (what Pointcloud.compute_pdf calls), reads whole lines instead."""
    d = _pdf_args("compute_pdf", bandwidth, pts, neigh, ends)
    out = torch.empty((pts.shape[0],), dtype=torch.float32, device=pts.device)
    _lib.call("pccnn_compute_pdf", int(manifold_dims), _ptr(bandwidth), _ptr(pts), pts.shape[0], d, _ptr(neigh),
              neigh.shape[0], _ptr(ends), _ptr(out), _stream())
    return out


def compute_pdf_sorted(manifold_dims, bandwidth, pts_sorted, samples, neigh_sorted, ends):
    """compute_pdf for a pair list in sorted-index space: column 0 of ``neigh_sorted`` indexes ``pts_sorted``,
    sample i is ``samples[i]``.  Returns f32[N] in the samples' order."""
    d = _pdf_args("compute_pdf_sorted", bandwidth, pts_sorted, neigh_sorted, ends)
    _chk(samples, "compute_pdf_sorted: samples", torch.float32, 2, pts_sorted.device)
    if tuple(samples.shape) != tuple(pts_sorted.shape):
        raise RuntimeError("compute_pdf_sorted: samples and pts_sorted must have the same shape")
    out = torch.empty((samples.shape[0],), dtype=torch.float32, device=samples.device)
    _lib.call("pccnn_compute_pdf_sorted", int(manifold_dims), _ptr(bandwidth), _ptr(pts_sorted), _ptr(samples),
              samples.shape[0], d, _ptr(neigh_sorted), neigh_sorted.shape[0], _ptr(ends), _ptr(out), _stream())
    return out


def compute_pdf_grid(manifold_dims, bandwidth, sorted_pts, sorted_keys, sample_order, grid_ds, grid_size, radii,
                     max_neighbors=0, cell_table=None, with_normalized=False):
    """The density of every point straight from the grid (no counterpart in the reference's module; it is what
    pccnn_lib/pc/Pointcloud.py:81-109 computes with find_neighbors + compute_pdf): sorted points f32[N,3], sorted
    keys i64[N], sample_order i32[N] (original index of sorted point i; None = the points already are in key
    order), pillar table, grid_size i32[3], radii f32[3] (the search radii = cell size) -> f32[N] in the original
    order, the same terms in the same order as compute_pdf on the (capped) neighbor list.  With
    ``with_normalized`` the result is the pair (estimate, estimate / number of points of the point's cloud)."""
    name = "compute_pdf_grid"
    _chk(sorted_pts, name + ": pts", torch.float32, 2)
    dev = sorted_pts.device
    _chk(bandwidth, name + ": bandwidth", torch.float32, 1, dev)
    _chk(sorted_keys, name + ": keys", torch.int64, 1, dev)
    _chk(grid_ds, name + ": grid_ds", torch.int32, 4, dev)
    _chk(grid_size, name + ": grid_size", torch.int32, 1, dev)
    _chk(radii, name + ": radii", torch.float32, 1, dev)
    n = sorted_pts.shape[0]
    if sorted_pts.shape[1] != 3 or sorted_keys.shape[0] != n or grid_size.shape[0] != 3 or radii.shape[0] != 3 \
            or bandwidth.shape[0] != 3 or grid_ds.shape[3] != 2:
        raise RuntimeError(name + ": 3-D points [N,3], keys [N], grid_ds [B,nc0,nc1,2], grid_size / radii / "
                                  "bandwidth [3]")
    max_neighbors = int(max_neighbors)
    if max_neighbors < 0:
        raise RuntimeError(name + ": max_neighbors must be >= 0")
    if sample_order is not None:
        _chk(sample_order, name + ": sample_order", torch.int32, 1, dev)
        if sample_order.shape[0] != n:
            raise RuntimeError(name + ": sample_order has the wrong length")
    total_cells = 0
    if cell_table is not None:
        _chk(cell_table, name + ": cell_table", torch.int32, 1, dev)
        total_cells = cell_table.shape[0] - 1
    out = torch.empty((n,), dtype=torch.float32, device=dev)
    norm = torch.empty_like(out) if with_normalized else None
    num_pillars = grid_ds.shape[0] * grid_ds.shape[1] * grid_ds.shape[2]
    _lib.call("pccnn_compute_pdf_grid", int(manifold_dims), _ptr(bandwidth), _ptr(sorted_pts), _ptr(sorted_keys), n,
              _optr(sample_order), _ptr(grid_ds), num_pillars, _optr(cell_table), total_cells, _ptr(grid_size),
              _ptr(radii), 3, max_neighbors, _ptr(out), _optr(norm), _stream())
    return (out, norm) if with_normalized else out


def pdf_cloud(manifold_dims, bandwidth, pts, batch_ids, aabb_min, cell_size, num_cells_host, batch_size,
              max_neighbors=0):
    """The density of every point of a 3-D cloud from its box and the grid size on the host: the grid of
    ``cell_size`` (the search radii) and the sum over it in one native call that only queues work (what
    pccnn_lib/pc/Pointcloud.py:81-109 computes; the kernels are those of ``grid_build`` and ``compute_pdf_grid``)
    -> (estimate f32[N], estimate / number of points of the point's cloud f32[N])."""
    name = "pdf_cloud"
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(bandwidth, name + ": bandwidth", torch.float32, 1, dev)
    _chk(batch_ids, name + ": batch_ids", torch.int32, 1, dev)
    _chk(aabb_min, name + ": aabb_min", torch.float32, 2, dev)
    _chk(cell_size, name + ": cell_size", torch.float32, 1, dev)
    n = pts.shape[0]
    batch_size = int(batch_size)
    max_neighbors = int(max_neighbors)
    if pts.shape[1] != 3 or batch_ids.shape[0] != n or tuple(aabb_min.shape) != (batch_size, 3) \
            or cell_size.shape[0] != 3 or bandwidth.shape[0] != 3 or max_neighbors < 0:
        raise RuntimeError(name + ": 3-D points [N,3], batch_ids [N], aabb_min [B,3], cell_size / bandwidth [3], "
                                  "three grid sizes, max_neighbors >= 0")
    out = torch.empty((2, n), dtype=torch.float32, device=dev)
    if n == 0:
        return out[0], out[1]
    cells = [int(v) for v in (num_cells_host() if callable(num_cells_host) else num_cells_host)]
    if len(cells) != 3 or min(cells) < 1:
        raise RuntimeError(name + ": three positive grid sizes")
    pillars = batch_size * cells[0] * cells[1]
    total = pillars * cells[2]
    with_table = 1 if total <= CELL_TABLE_MAX_CELLS else 0
    ws = _workspace(_lib.load().pccnn_pdf_cloud_workspace_bytes(n, pillars, total if with_table else 0), dev)
    base = out.data_ptr()
    _lib.call("pccnn_pdf_cloud", int(manifold_dims), _ptr(bandwidth), _ptr(pts), _ptr(batch_ids), n, batch_size,
              _ptr(aabb_min), _ptr(cell_size), (ctypes.c_int32 * 3)(*cells), key_bits_for(cells, batch_size), with_table,
              max_neighbors, _P(base), _P(base + 4 * n), _ptr(ws), ws.numel(), _stream())
    return out[0], out[1]


def compute_pdf_grads(manifold_dims, bandwidth, pts, neigh, ends, in_grads):
    """compute_pdf_grads(..., in_grads f32[N]) -> f32[N,D] (pccnn_lib_ops/compute_pdf/compute_pdf.cuh:45-51)."""
    d = _pdf_args("compute_pdf_grads", bandwidth, pts, neigh, ends)
    in_grads = _chk(in_grads.contiguous(), "compute_pdf_grads: in_grads", torch.float32, 1, pts.device)
    if in_grads.shape[0] != pts.shape[0]:
        raise RuntimeError("compute_pdf_grads: in_grads has the wrong length")
    out = torch.empty_like(pts)
    _lib.call("pccnn_compute_pdf_grads", int(manifold_dims), _ptr(bandwidth), _ptr(pts), pts.shape[0], d, _ptr(neigh),
              neigh.shape[0], _ptr(ends), _ptr(in_grads), _ptr(out), _stream())
    return out


# -------------------------------------------------------------------------- pooling


def poisson_disk_sampling(sorted_keys, neigh, ends, grid_size):
    """poisson_disk_sampling(sorted keys i64[N], neighbors, start_ids, grid_size) -> i64[S,1], all in sorted-index
    space (pccnn_lib_ops/poisson_disk_sampling/poisson_disk_sampling.cuh:28-32)."""
    name = "poisson_disk_sampling"
    _chk(sorted_keys, name + ": keys", torch.int64, 1)
    dev = sorted_keys.device
    _chk(neigh, name + ": neighbors", torch.int32, 2, dev)
    _chk(ends, name + ": start_ids", torch.int32, 1, dev)
    _chk(grid_size, name + ": grid_size", torch.int32, 1, dev)
    n = sorted_keys.shape[0]
    d = grid_size.shape[0]
    if ends.shape[0] != n or d < MIN_DIMS or d > MAX_DIMS or neigh.shape[1] != 2:
        raise RuntimeError(name + ": inconsistent shapes")
    if n == 0:
        return torch.empty((0, 1), dtype=torch.int64, device=dev)
    sel = torch.empty((n,), dtype=torch.int32, device=dev)
    scan = torch.empty_like(sel)
    ws = _workspace(_lib.load().pccnn_poisson_disk_workspace_bytes(n), dev)
    _lib.call("pccnn_poisson_disk_select", _ptr(sorted_keys), n, _ptr(neigh), neigh.shape[0], _ptr(ends),
              _ptr(grid_size), d, _ptr(sel), _ptr(scan), _ptr(ws), ws.numel(), _stream())
    count = int(scan[-1].item())
    ids = torch.empty((count, 1), dtype=torch.int64, device=dev)
    _lib.call("pccnn_compact_selected", _ptr(sel), _ptr(scan), n, _ptr(ids), _stream())
    return ids


def poisson_disk_sampling_grid(sorted_pts, sorted_keys, grid_ds, grid_size, radii, cell_table=None):
    """Poisson-disk selection straight from the grid (no counterpart in the reference's module; it is what
    pccnn_lib/pc/PointPooling.py:58-65 computes with find_neighbors + poisson_disk_sampling): sorted points
    f32[N,3], sorted keys i64[N], pillar table, grid_size i32[3], radii f32[3] (= the cell size) -> i64[S,1] in
    sorted-index space, identical to poisson_disk_sampling on the uncapped self-neighborhood."""
    name = "poisson_disk_sampling_grid"
    _chk(sorted_pts, name + ": pts", torch.float32, 2)
    dev = sorted_pts.device
    _chk(sorted_keys, name + ": keys", torch.int64, 1, dev)
    _chk(grid_ds, name + ": grid_ds", torch.int32, 4, dev)
    _chk(grid_size, name + ": grid_size", torch.int32, 1, dev)
    _chk(radii, name + ": radii", torch.float32, 1, dev)
    n = sorted_pts.shape[0]
    if sorted_pts.shape[1] != 3 or sorted_keys.shape[0] != n or grid_size.shape[0] != 3 or radii.shape[0] != 3 \
            or grid_ds.shape[3] != 2:
        raise RuntimeError(name + ": 3-D points [N,3], keys [N], grid_ds [B,nc0,nc1,2], grid_size [3], radii [3]")
    if n == 0:
        return torch.empty((0, 1), dtype=torch.int64, device=dev)
    total_cells = 0
    if cell_table is not None:
        _chk(cell_table, name + ": cell_table", torch.int32, 1, dev)
        total_cells = cell_table.shape[0] - 1
    sel = torch.empty((n,), dtype=torch.int32, device=dev)
    scan = torch.empty_like(sel)
    ws = _workspace(_lib.load().pccnn_poisson_disk_workspace_bytes(n), dev)
    num_pillars = grid_ds.shape[0] * grid_ds.shape[1] * grid_ds.shape[2]
    _lib.call("pccnn_poisson_disk_grid", _ptr(sorted_pts), _ptr(sorted_keys), n, _ptr(grid_ds), num_pillars,
              _optr(cell_table), total_cells, _ptr(grid_size), _ptr(radii), 3, _ptr(sel), _ptr(scan), _ptr(ws),
              ws.numel(), _stream())
    count = int(scan[-1].item())
    ids = torch.empty((count, 1), dtype=torch.int64, device=dev)
    _lib.call("pccnn_compact_selected", _ptr(sel), _ptr(scan), n, _ptr(ids), _stream())
    return ids


def pool_poisson(pts, batch_ids, aabb_min, cell_size, num_cells_host, batch_size):
    """Poisson-disk pooling of a 3-D cloud from its box and the grid size on the host (what
    pccnn_lib/pc/PointPooling.py:38-69 does after the bounding box): the grid, the selection and its size in one
    native call, the selected points' ORIGINAL indices, coordinates and batch ids in a second one -> (i64[S] in key
    order, box, f32[S,3], i32[S]), where box =
    (min f32[B,3], max f32[B,3], (numpy min, numpy max)) is the bounding box of the selected points per cloud, as
    ``bounding_box_host`` of the pooled cloud would return it (it comes back with the count, in the same read).
    No counterpart in the reference's module; the kernels are those of grid_build, poisson_disk_sampling_grid and
    bounding_box."""
    return pool_poisson_later(pts, batch_ids, aabb_min, cell_size, num_cells_host, batch_size)()


def pool_poisson_later(pts, batch_ids, aabb_min, cell_size, num_cells_host, batch_size):
    """``pool_poisson`` in two halves: the call queues grid, selection, box and the copy of count and box to pinned
    memory and returns ``finish``; ``finish()`` waits for that copy, gathers the selected rows and returns what
    ``pool_poisson`` returns.  Work the caller queues between the two (the cloud's density, say) runs on the device
    while the host waits for the count."""
    import numpy as np
    name = "pool_poisson"
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(batch_ids, name + ": batch_ids", torch.int32, 1, dev)
    _chk(aabb_min, name + ": aabb_min", torch.float32, 2, dev)
    _chk(cell_size, name + ": cell_size", torch.float32, 1, dev)
    n = pts.shape[0]
    batch_size = int(batch_size)
    if pts.shape[1] != 3 or batch_ids.shape[0] != n or tuple(aabb_min.shape) != (batch_size, 3) \
            or cell_size.shape[0] != 3:
        raise RuntimeError(name + ": 3-D points [N,3], batch_ids [N], aabb_min [B,3], cell_size [3], three grid sizes")
    if n == 0:
        empty = (torch.empty((0,), dtype=torch.int64, device=dev), None, torch.empty_like(pts),
                 torch.empty_like(batch_ids))
        finish = lambda: empty
        finish.wait = lambda: None
        return finish
    lib = _lib.load()
    rows = torch.empty((3 * n,), dtype=torch.int32, device=dev)      # permutation | selection flags | their scan
    base = rows.data_ptr()
    box = torch.empty((2, batch_size, 3), dtype=torch.float32, device=dev)
    landing = torch.empty((6 * batch_size + 1,), dtype=torch.float32, pin_memory=True)
    words = landing.numpy().view(np.int32)
    words[6 * batch_size] = -1                                     # the count arrives last: polled below
    # (the grid size last: when it is a callable it may have to wait for the cloud's box to arrive on the host)
    cells = [int(v) for v in (num_cells_host() if callable(num_cells_host) else num_cells_host)]
    if len(cells) != 3 or min(cells) < 1:
        raise RuntimeError(name + ": three positive grid sizes")
    pillars = batch_size * cells[0] * cells[1]
    total = pillars * cells[2]
    with_table = 1 if total <= CELL_TABLE_MAX_CELLS else 0
    ws = _workspace(lib.pccnn_pool_poisson_workspace_bytes(n, pillars, total if with_table else 0), dev)
    polled = ctypes.c_int(0)
    _lib.call("pccnn_pool_poisson_select_queued", _ptr(pts), _ptr(batch_ids), n, batch_size, _ptr(aabb_min),
              _ptr(cell_size), (ctypes.c_int32 * 3)(*cells), key_bits_for(cells, batch_size), with_table, _P(base),
              _P(base + 4 * n), _P(base + 8 * n), _P(box.data_ptr()), _P(box.data_ptr() + 12 * batch_size),
              _P(landing.data_ptr()), ctypes.byref(polled), _ptr(ws), ws.numel(), _stream())
    done = torch.cuda.Event()
    done.record()
    _keep_until_written(landing, done)

    def finish():
        # written by the kernels: the count is the last word to arrive, so a short poll of the pinned word, then
        # the event if it takes long; brought over by copies (many clouds): the event right away
        spins = 0
        while polled.value and words[6 * batch_size] < 0:
            spins += 1
            if spins > SPIN_LIMIT:
                break
        if words[6 * batch_size] < 0:
            done.synchronize()
        host = landing.numpy()
        count = int(words[6 * batch_size])
        if count < 0:
            raise RuntimeError(name + ": the selection's size did not arrive")
        host_box = host[:6 * batch_size].reshape(2, batch_size, 3)
        ids = torch.empty((count,), dtype=torch.int64, device=dev)
        pooled_pts = torch.empty((count, 3), dtype=torch.float32, device=dev)
        pooled_ids = torch.empty((count,), dtype=torch.int32, device=dev)
        # (`rows` through the tensor itself: the closure keeps permutation, flags and scan alive until they are read)
        at = rows.data_ptr()
        _lib.call("pccnn_compact_pooled", _P(at + 4 * n), _P(at + 8 * n), _P(at), _ptr(pts), _ptr(batch_ids), n,
                  3, _ptr(ids), _ptr(pooled_pts), _ptr(pooled_ids), _stream())
        return ids, (box[0], box[1], (host_box[0], host_box[1])), pooled_pts, pooled_ids
    # a caller that drops `finish` unused waits with this before it lets go of it: the copy into the pinned block
    # must have landed before the block can be handed out again
    finish.wait = done.synchronize
    finish.polled = bool(polled.value)
    return finish


# ----------------------------------------------------------------------------- conv

# Gradient groups of the backward entry points (PCCNN_GRAD_* in include/pccnn_hip.h).
GRAD_WEIGHTS, GRAD_FEATS, GRAD_BASIS_PARAMS, GRAD_PDF, GRAD_PTS, GRAD_ALL = 1, 2, 4, 8, 16, 31
# Flag beside the groups: the backward pass without float atomics (bit-identical results from run to run, slower).
GRAD_DETERMINISTIC = 32

_deterministic = False


def set_deterministic(on):
    """``set_deterministic(True)``: the autograd wrappers ask the backward calls for the pass without float atomics
    (``GRAD_DETERMINISTIC``), so gradients are bit-identical from run to run.  Returns the previous setting."""
    global _deterministic
    before, _deterministic = _deterministic, bool(on)
    return before


def deterministic_flag():
    """``GRAD_DETERMINISTIC`` while ``set_deterministic(True)`` is in force, else 0: OR it into a grad_mask."""
    return GRAD_DETERMINISTIC if _deterministic else 0


def _backward_workspace(n, m, t, c_in, k, c_out, grad_mask, dev, mirror=None):
    """Workspace of a backward call: the larger one when the pass without atomics is asked for, and when the library
    may take the per-pair rows by itself (a mirror index, wide rows, no basis / position / density gradients)."""
    lib = _lib.load()
    rows_route = mirror is not None and c_in > 32 and not (grad_mask & (GRAD_BASIS_PARAMS | GRAD_PDF | GRAD_PTS))
    if grad_mask & GRAD_DETERMINISTIC or (rows_route and grad_mask & GRAD_FEATS):
        return _workspace(lib.pccnn_conv_workspace_bytes_deterministic(n, m, t, c_in, k, c_out), dev)
    return _workspace(lib.pccnn_conv_workspace_bytes(m, t, c_in, k, c_out, 1), dev)



def _conv_dims(pts, name, only_3d=False):
    d = pts.shape[1]
    if d < MIN_DIMS or d > MAX_DIMS or (only_3d and d != 3):
        raise RuntimeError("%s: %d-dimensional points are not supported (%s)"
                           % (name, d, "3 only" if only_3d else "%d to %d" % (MIN_DIMS, MAX_DIMS)))
    return d


def _forward_workspace(pts, m, t, c_in, k, c_out, dev, keep_proj=True):
    """(pointer, bytes) of the forward call's workspace: clouds that are not 3-D need one for the per-pair basis, and
    a call that does not keep the projection needs one for it (or, when the library keeps the projection on chip,
    for the repacked weights).  Returns the tensor too, to keep it alive over the call."""
    if keep_proj and (pts is None or pts.shape[1] == 3):
        return _P(0), 0, None
    ws = _workspace(_lib.load().pccnn_conv_workspace_bytes(m, t, c_in, k, c_out, 0), dev)
    return _ptr(ws), ws.numel(), ws


def _dims_of(pts):
    """Dimension argument of the generic entry points; a caller-given basis has no geometry."""
    return 3 if pts is None else pts.shape[1]


# Planar clouds run through the 3-D kernels with a zero third coordinate: positions, samples and kernel points get
# a zero column, axis matrices a zero row, the radii a 1; every term the extra coordinate adds is an exact zero, so
# the results are those of the 2-D formulas, and the extra gradient components are dropped.
def _is_planar(pts):
    return isinstance(pts, torch.Tensor) and pts.dim() == 2 and pts.shape[1] == 2


def _pad_cols(x, value=0.0):
    """[n, 2] -> [n, 3] (or [2] -> [3])."""
    return torch.nn.functional.pad(x, (0, 1), value=value).contiguous()


def _pad_rows(x):
    """[2, k] -> [3, k]."""
    return torch.nn.functional.pad(x, (0, 0, 0, 1)).contiguous()


def _cut(x):
    return None if x is None else x[:, :2].contiguous()


def _conv_args(name, pts, feats, samples, neigh, ends, radii):
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    _chk(feats, name + ": features", torch.float32, 2, dev)
    _chk(samples, name + ": samples", torch.float32, 2, dev)
    _chk(neigh, name + ": neighbors", torch.int32, 2, dev)
    _chk(ends, name + ": start_ids", torch.int32, 1, dev)
    _chk(radii, name + ": radii", torch.float32, 1, dev)
    d = _conv_dims(pts, name)
    if feats.shape[0] != pts.shape[0] or samples.shape[1] != d or ends.shape[0] != samples.shape[0] \
            or neigh.shape[1] != 2 or radii.shape[0] != d:
        raise RuntimeError(name + ": inconsistent shapes")
    return d, dev


def kp_conv(pts, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, return_proj=False,
            contraction="f32"):
    """kp_conv(pts, feats, samples, neighbors, start_ids, radii, kernel_pts f32[K,D], sigma, weights f32[K*Cin,Cout])
    -> f32[M,Cout] (pccnn_lib_ops/pcconvs/kpconv.cuh:32-41).  ``return_proj=True`` also returns the projection
    f32[M,Cin,K] the call built, for kp_conv_grads(..., proj=...).  ``contraction="bf16"`` (no counterpart in the
    reference) rounds the operands of the [M,K*Cin] x [K*Cin,Cout] product to bf16 and accumulates in fp32; the
    projection returned is then bf16."""
    name = "kp_conv"
    if _is_planar(pts):
        return kp_conv(_pad_cols(pts), feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                       _pad_cols(kernel_pts), sigma, weights, return_proj, contraction)
    bf16 = _contraction(name, contraction)
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    _chk(kernel_pts, name + ": kernel_pts", torch.float32, 2, dev)
    _chk(weights, name + ": weights", torch.float32, 2, dev)
    n, m, t, c_in, k, c_out = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1], kernel_pts.shape[0], \
        weights.shape[1]
    if kernel_pts.shape[1] != d or weights.shape[0] != k * c_in:
        raise RuntimeError(name + ": weights must be [K*Cin, Cout] and kernel_pts [K, D]")
    if bf16:
        desc = _basis(BASIS_KP, k, a=kernel_pts, sigma=sigma)
        out, proj = _bf16_forward(name, desc, pts, feats, samples, neigh, ends, radii, weights, k, 1, c_out,
                                  return_proj)
        return (out, proj) if return_proj else out
    out = torch.empty((m, c_out), dtype=torch.float32, device=dev)
    proj = torch.empty((m, c_in, k), dtype=torch.float32, device=dev) if return_proj else None
    ws_p, ws_n, _ws = _forward_workspace(pts, m, t, c_in, k, c_out, dev, return_proj)
    _lib.call("pccnn_kpconv_forward", _ptr(pts), _ptr(feats), _ptr(samples), _ptr(neigh), _ptr(ends), _ptr(radii),
              _ptr(kernel_pts), float(sigma), _ptr(weights), n, m, t, d, c_in, k, c_out, _ptr(out), _optr(proj),
              ws_p, ws_n, _stream())
    return (out, proj) if return_proj else out


def _bf16_forward(name, desc, pts, feats, samples, neigh, ends, radii, weights, k, num_mlps, c_out, keep_proj=True):
    """Forward call with the contraction operands in bf16; returns (out f32[M,Cout], proj bf16[M,Cin,K] or None)."""
    dev = feats.device
    n, m, t, c_in = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1]
    out = torch.empty((m, c_out), dtype=torch.float32, device=dev)
    proj = torch.empty((m, c_in, k), dtype=torch.bfloat16, device=dev) if keep_proj else None
    ws = _workspace(_lib.load().pccnn_conv_workspace_bytes(m, t, c_in, k, c_out, 0), dev)
    _lib.call("pccnn_conv_forward_bf16", ctypes.byref(desc), _ptr(pts), _ptr(feats), _ptr(samples), _ptr(neigh),
              _ptr(ends), _ptr(radii), _ptr(weights), n, m, t, _dims_of(pts), c_in, num_mlps, c_out, 0, _ptr(out),
              _optr(proj), _ptr(ws), ws.numel(), _stream())
    return out, proj


def _bf16_backward(name, desc, pts, feats, samples, neigh, ends, radii, weights, in_grads, proj, mirror, grad_mask,
                   k, num_mlps, c_out, d_w, d_f, d_a, d_b, d_pdf, d_p, d_s):
    dev = feats.device
    n, m, t, c_in = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1]
    proj_p = _conv_proj_arg(name, proj, m, c_in, k, dev, bf16=True)
    ws = _backward_workspace(n, m, t, c_in, k, c_out, grad_mask, dev, mirror)
    _lib.call("pccnn_conv_backward_bf16", ctypes.byref(desc), _ptr(pts), _ptr(feats), _ptr(samples), _ptr(neigh),
              _ptr(ends), _ptr(radii), _ptr(weights), _ptr(in_grads), proj_p,
              _mirror_arg(name, mirror, neigh, pts, samples), grad_mask, n, m, t, _dims_of(pts), c_in, num_mlps, c_out, 0,
              _optr(d_w), _optr(d_f), _optr(d_a), _optr(d_b), _optr(d_pdf), _optr(d_p), _optr(d_s), _ptr(ws),
              ws.numel(), _stream())


def _mirror_arg(name, mirror, neigh, pts, samples):
    if mirror is None:
        return _P(0)
    _chk(mirror, name + ": mirror", torch.int32, 1, neigh.device)
    if mirror.shape[0] != neigh.shape[0] or pts.shape[0] != samples.shape[0]:
        raise RuntimeError(name + ": mirror must be [T] and needs samples == points")
    return _ptr(mirror)


def gather_rows(rows, index):
    """rows[index] for float32 rows [N] or [N, C] and an int32 index [M] (no counterpart in the reference op module;
    what its Python does with torch.index_select)."""
    _chk(rows, "gather_rows: rows", torch.float32)
    _chk(index, "gather_rows: index", torch.int32, 1, rows.device)
    width = 1
    for extent in rows.shape[1:]:
        width *= int(extent)
    out = torch.empty((index.shape[0],) + tuple(rows.shape[1:]), dtype=torch.float32, device=rows.device)
    if index.shape[0] > 0 and width > 0:
        if rows.shape[0] == 0:
            raise RuntimeError("gather_rows: an index into an empty tensor")
        _lib.call("pccnn_gather_rows_f32", _ptr(rows), _ptr(index), _ptr(out), index.shape[0], width, rows.shape[0],
                  _stream())
    return out


def invert_permutation(perm):
    """int32 [N] with inverse[perm[i]] = i, for a permutation of 0 .. N-1."""
    _chk(perm, "invert_permutation: perm", torch.int32, 1)
    inverse = torch.empty_like(perm)
    _lib.call("pccnn_invert_permutation_i32", _ptr(perm), _ptr(inverse), perm.shape[0], _stream())
    return inverse


def mirror_pairs(neigh, ends):
    """Mirror index of a symmetric neighborhood (samples are the points, uncapped search): int32 [T] with the
    index of pair (b, a) for every pair (a, b), or None when some pair has no mirror.  Reads one int back."""
    _chk(neigh, "mirror_pairs: neighbors", torch.int32, 2)
    _chk(ends, "mirror_pairs: start_ids", torch.int32, 1, neigh.device)
    mirror = torch.empty((neigh.shape[0],), dtype=torch.int32, device=neigh.device)
    missing = torch.empty((1,), dtype=torch.int32, device=neigh.device)
    _lib.call("pccnn_mirror_pairs", _ptr(neigh), _ptr(ends), neigh.shape[0], ends.shape[0], _ptr(mirror),
              _ptr(missing), _stream())
    return mirror if int(missing.item()) == 0 else None


def kp_conv_grads(pts, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, in_grads, proj=None,
                  grad_mask=GRAD_ALL, mirror=None, contraction="f32"):
    """kp_conv_grads(..., in_grads f32[M,Cout]) -> [dW, dFeat, dKernelPts, dPts, dSamples]
    (pccnn_lib_ops/pcconvs/kpconv.cuh:56-67).  ``proj``: projection kept from kp_conv(return_proj=True);
    ``grad_mask``: GRAD_* groups to compute, the others come back as None; ``mirror``: result of mirror_pairs()
    for a symmetric neighborhood, which lets dPts (and dPdf) be summed per point without atomics."""
    name = "kp_conv_grads"
    if _is_planar(pts):
        d_w, d_f, d_kp, d_p, d_s = kp_conv_grads(_pad_cols(pts), feats, _pad_cols(samples), neigh, ends,
                                                 _pad_cols(radii, 1.0), _pad_cols(kernel_pts), sigma, weights, in_grads,
                                                 proj, grad_mask, mirror, contraction)
        return [d_w, d_f, _cut(d_kp), _cut(d_p), _cut(d_s)]
    bf16 = _contraction(name, contraction)
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    _chk(kernel_pts, name + ": kernel_pts", torch.float32, 2, dev)
    _chk(weights, name + ": weights", torch.float32, 2, dev)
    in_grads = _chk(in_grads.contiguous(), name + ": in_grads", torch.float32, 2, dev)
    n, m, t, c_in, k, c_out = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1], kernel_pts.shape[0], \
        weights.shape[1]
    if kernel_pts.shape[1] != d or weights.shape[0] != k * c_in or tuple(in_grads.shape) != (m, c_out):
        raise RuntimeError(name + ": inconsistent shapes")
    grad_mask = int(grad_mask)
    alloc = lambda like, bit: torch.empty_like(like) if grad_mask & bit else None
    d_w, d_f, d_kp = alloc(weights, GRAD_WEIGHTS), alloc(feats, GRAD_FEATS), alloc(kernel_pts, GRAD_BASIS_PARAMS)
    d_p, d_s = alloc(pts, GRAD_PTS), alloc(samples, GRAD_PTS)
    if bf16:
        desc = _basis(BASIS_KP, k, a=kernel_pts, sigma=sigma)
        _bf16_backward(name, desc, pts, feats, samples, neigh, ends, radii, weights, in_grads, proj, mirror, grad_mask,
                       k, 1, c_out, d_w, d_f, d_kp, None, None, d_p, d_s)
        return [d_w, d_f, d_kp, d_p, d_s]
    proj_p = _conv_proj_arg(name, proj, m, c_in, k, dev)
    ws = _backward_workspace(n, m, t, c_in, k, c_out, grad_mask, dev, mirror)
    _lib.call("pccnn_kpconv_backward", _ptr(pts), _ptr(feats), _ptr(samples), _ptr(neigh), _ptr(ends), _ptr(radii),
              _ptr(kernel_pts), float(sigma), _ptr(weights), _ptr(in_grads), proj_p,
              _mirror_arg(name, mirror, neigh, pts, samples), grad_mask, n, m, t, d, c_in, k,
              c_out, _optr(d_w), _optr(d_f), _optr(d_kp), _optr(d_p), _optr(d_s), _ptr(ws), ws.numel(), _stream())
    return [d_w, d_f, d_kp, d_p, d_s]


def _optr(t):
    return _P(t.data_ptr()) if t is not None else _P(0)


CONTRACTIONS = ("f32", "bf16")


def _contraction(name, contraction):
    if contraction not in CONTRACTIONS:
        raise RuntimeError("%s: contraction must be one of %s, got %r" % (name, CONTRACTIONS, contraction))
    return contraction == "bf16"


def _conv_proj_arg(name, proj, m, c_in, k, dev, bf16=False):
    if proj is None:
        return _P(0)
    _chk(proj, name + ": proj", torch.bfloat16 if bf16 else torch.float32, 3, dev)
    if tuple(proj.shape) != (m, c_in, k):
        raise RuntimeError(name + ": proj must be [M, Cin, K]")
    return _ptr(proj)


def _mc_args(name, pts, pdf, axis, bias, weights, c_in, d, dev):
    _chk(pdf, name + ": pdf", torch.float32, 1, dev)
    _chk(axis, name + ": axis", torch.float32, 2, dev)
    _chk(bias, name + ": bias", torch.float32, 2, dev)
    _chk(weights, name + ": weights", torch.float32, 3, dev)
    k = axis.shape[1]
    num_mlps, c_out = weights.shape[0], weights.shape[0] * weights.shape[2]
    if pdf.shape[0] != pts.shape[0] or axis.shape[0] != d or tuple(bias.shape) != (1, k) \
            or weights.shape[1] * num_mlps != k * c_in:
        raise RuntimeError(name + ": axis must be [D, H*mlps], bias [1, H*mlps], weights [mlps, H*Cin, Cout/mlps]")
    return k, num_mlps, c_out


def mc_conv(pts, pdf, feats, samples, neigh, ends, radii, axis, bias, weights, return_proj=False,
            contraction="f32"):
    """mc_conv(pts, pdf f32[N], feats, samples, neighbors, start_ids, radii, axis f32[D,H*m], bias f32[1,H*m],
    weights f32[m, H*Cin, Cout/m]) -> f32[M,Cout] (pccnn_lib_ops/pcconvs/mcconv.cuh:32-42).
    ``return_proj=True`` also returns the projection f32[M,Cin,H*m] for mc_conv_grads(..., proj=...);
    ``contraction`` as in kp_conv."""
    name = "mc_conv"
    if _is_planar(pts):
        return mc_conv(_pad_cols(pts), pdf, feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                       _pad_rows(axis), bias, weights, return_proj, contraction)
    bf16 = _contraction(name, contraction)
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    n, m, t, c_in = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1]
    k, num_mlps, c_out = _mc_args(name, pts, pdf, axis, bias, weights, c_in, d, dev)
    if bf16:
        desc = _basis(BASIS_MLP, k, a=axis, b=bias, pdf=pdf)
        out, proj = _bf16_forward(name, desc, pts, feats, samples, neigh, ends, radii, weights, k, num_mlps, c_out,
                                  return_proj)
        return (out, proj) if return_proj else out
    out = torch.empty((m, c_out), dtype=torch.float32, device=dev)
    proj = torch.empty((m, c_in, k), dtype=torch.float32, device=dev) if return_proj else None
    ws_p, ws_n, _ws = _forward_workspace(pts, m, t, c_in, k, c_out, dev, return_proj)
    _lib.call("pccnn_mcconv_forward", _ptr(pts), _ptr(pdf), _ptr(feats), _ptr(samples), _ptr(neigh), _ptr(ends),
              _ptr(radii), _ptr(axis), _ptr(bias), _ptr(weights), n, m, t, d, c_in, k, num_mlps, c_out, _ptr(out),
              _optr(proj), ws_p, ws_n, _stream())
    return (out, proj) if return_proj else out


def mc_conv_grads(pts, pdf, feats, samples, neigh, ends, radii, axis, bias, weights, in_grads, proj=None,
                  grad_mask=GRAD_ALL, mirror=None, contraction="f32"):
    """mc_conv_grads(..., in_grads f32[M,Cout]) -> [dW, dFeat, dAxis, dBias f32[1,H*m], dPdf f32[N], dPts, dSamples]
    (pccnn_lib_ops/pcconvs/mcconv.cuh:57-69).  ``proj`` / ``grad_mask`` / ``mirror`` as in kp_conv_grads."""
    name = "mc_conv_grads"
    if _is_planar(pts):
        g = mc_conv_grads(_pad_cols(pts), pdf, feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                          _pad_rows(axis), bias, weights, in_grads, proj, grad_mask, mirror, contraction)
        return [g[0], g[1], None if g[2] is None else g[2][:2].contiguous(), g[3], g[4], _cut(g[5]), _cut(g[6])]
    bf16 = _contraction(name, contraction)
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    n, m, t, c_in = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1]
    k, num_mlps, c_out = _mc_args(name, pts, pdf, axis, bias, weights, c_in, d, dev)
    in_grads = _chk(in_grads.contiguous(), name + ": in_grads", torch.float32, 2, dev)
    if tuple(in_grads.shape) != (m, c_out):
        raise RuntimeError(name + ": in_grads must be [M, Cout]")
    grad_mask = int(grad_mask)
    alloc = lambda like, bit: torch.empty_like(like) if grad_mask & bit else None
    d_w, d_f = alloc(weights, GRAD_WEIGHTS), alloc(feats, GRAD_FEATS)
    d_axis, d_bias, d_pdf = alloc(axis, GRAD_BASIS_PARAMS), alloc(bias, GRAD_BASIS_PARAMS), alloc(pdf, GRAD_PDF)
    d_p, d_s = alloc(pts, GRAD_PTS), alloc(samples, GRAD_PTS)
    if bf16:
        desc = _basis(BASIS_MLP, k, a=axis, b=bias, pdf=pdf)
        _bf16_backward(name, desc, pts, feats, samples, neigh, ends, radii, weights, in_grads, proj, mirror, grad_mask,
                       k, num_mlps, c_out, d_w, d_f, d_axis, d_bias, d_pdf, d_p, d_s)
        return [d_w, d_f, d_axis, d_bias, d_pdf, d_p, d_s]
    proj_p = _conv_proj_arg(name, proj, m, c_in, k, dev)
    ws = _backward_workspace(n, m, t, c_in, k, c_out, grad_mask, dev, mirror)
    _lib.call("pccnn_mcconv_backward", _ptr(pts), _ptr(pdf), _ptr(feats), _ptr(samples), _ptr(neigh), _ptr(ends),
              _ptr(radii), _ptr(axis), _ptr(bias), _ptr(weights), _ptr(in_grads), proj_p,
              _mirror_arg(name, mirror, neigh, pts, samples), grad_mask, n, m, t, d, c_in, k, num_mlps, c_out, _optr(d_w), _optr(d_f), _optr(d_axis), _optr(d_bias), _optr(d_pdf), _optr(d_p),
              _optr(d_s), _ptr(ws), ws.numel(), _stream())
    return [d_w, d_f, d_axis, d_bias, d_pdf, d_p, d_s]


def kp_conv_weight_var(pts, feats, samples, neigh, ends, radii, kernel_pts, sigma):
    """kp_conv_weight_var(pts, feats, samples, neighbors, start_ids, radii, kernel_pts, sigma) -> 0-d float tensor
    (pccnn_lib_ops/pcconvs/kpconv.cuh:82-90)."""
    name = "kp_conv_weight_var"
    if _is_planar(pts):
        return kp_conv_weight_var(_pad_cols(pts), feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                                  _pad_cols(kernel_pts), sigma)
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    _chk(kernel_pts, name + ": kernel_pts", torch.float32, 2, dev)
    n, m, t, c_in, k = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1], kernel_pts.shape[0]
    if kernel_pts.shape[1] != d:
        raise RuntimeError(name + ": kernel_pts must be [K, D]")
    out = torch.empty((1,), dtype=torch.float32, device=dev)
    ws = _workspace(_lib.load().pccnn_conv_weight_var_workspace_bytes(m, t, c_in, k), dev)
    _lib.call("pccnn_kpconv_weight_var", _ptr(pts), _ptr(feats), _ptr(samples), _ptr(neigh), _ptr(ends), _ptr(radii),
              _ptr(kernel_pts), float(sigma), n, m, t, d, c_in, k, _ptr(out), _ptr(ws), ws.numel(), _stream())
    return out.reshape(())


def mc_conv_weight_var(pts, pdf, feats, samples, neigh, ends, radii, axis, bias):
    """mc_conv_weight_var(pts, pdf, feats, samples, neighbors, start_ids, radii, axis, bias) -> 0-d float tensor
    (pccnn_lib_ops/pcconvs/mcconv.cuh:83-92)."""
    name = "mc_conv_weight_var"
    if _is_planar(pts):
        return mc_conv_weight_var(_pad_cols(pts), pdf, feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                                  _pad_rows(axis), bias)
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    _chk(pdf, name + ": pdf", torch.float32, 1, dev)
    _chk(axis, name + ": axis", torch.float32, 2, dev)
    _chk(bias, name + ": bias", torch.float32, 2, dev)
    n, m, t, c_in, k = pts.shape[0], samples.shape[0], neigh.shape[0], feats.shape[1], axis.shape[1]
    if pdf.shape[0] != n or axis.shape[0] != d or tuple(bias.shape) != (1, k):
        raise RuntimeError(name + ": axis must be [D, H*mlps], bias [1, H*mlps], pdf [N]")
    out = torch.empty((1,), dtype=torch.float32, device=dev)
    ws = _workspace(_lib.load().pccnn_conv_weight_var_workspace_bytes(m, t, c_in, k), dev)
    _lib.call("pccnn_mcconv_weight_var", _ptr(pts), _ptr(pdf), _ptr(feats), _ptr(samples), _ptr(neigh), _ptr(ends),
              _ptr(radii), _ptr(axis), _ptr(bias), n, m, t, d, c_in, k, _ptr(out), _ptr(ws), ws.numel(), _stream())
    return out.reshape(())


# ------------------------------------------------- the other convolution families

BASIS_KP, BASIS_MLP, BASIS_KPN, BASIS_GAUSS, BASIS_EXPLICIT, BASIS_SPH = range(6)


def _basis(kind, k=0, a=None, b=None, c=None, sigma=1.0, pdf=None):
    """struct pccnn_basis for one call; the tensors it points to must stay alive until the call returns."""
    desc = _lib.Basis()
    desc.kind, desc.k, desc.sigma = kind, k, float(sigma)
    desc.a, desc.b, desc.c, desc.pdf = (None if x is None else x.data_ptr() for x in (a, b, c, pdf))
    if kind == BASIS_SPH:
        desc.nb0, desc.nb1, desc.nb2 = a.shape[0], b.shape[0], c.shape[0]
    return desc


def _generic_forward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, divide_by_count, return_proj):
    dev = feats.device
    _chk(weights, name + ": weights", torch.float32, 2, dev)
    n, m, t, c_in, c_out = feats.shape[0], ends.shape[0], neigh.shape[0], feats.shape[1], weights.shape[1]
    if weights.shape[0] != k * c_in:
        raise RuntimeError(name + ": weights must be [K*Cin, Cout]")
    out = torch.empty((m, c_out), dtype=torch.float32, device=dev)
    proj = torch.empty((m, c_in, k), dtype=torch.float32, device=dev) if return_proj else None
    ws_p, ws_n, _ws = _forward_workspace(pts, m, t, c_in, k, c_out, dev, return_proj)
    _lib.call("pccnn_conv_forward", ctypes.byref(desc), _optr(pts), _ptr(feats), _optr(samples), _ptr(neigh),
              _ptr(ends), _optr(radii), _ptr(weights), n, m, t, _dims_of(pts), c_in, 1, c_out, int(divide_by_count),
              _ptr(out), _optr(proj), ws_p, ws_n, _stream())
    return (out, proj) if return_proj else out


def _generic_backward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, in_grads, proj, grad_mask,
                      divide_by_count, d_param_a=None, d_pdf=None, with_pts=True, mirror=None):
    dev = feats.device
    _chk(weights, name + ": weights", torch.float32, 2, dev)
    in_grads = _chk(in_grads.contiguous(), name + ": in_grads", torch.float32, 2, dev)
    n, m, t, c_in, c_out = feats.shape[0], ends.shape[0], neigh.shape[0], feats.shape[1], weights.shape[1]
    if weights.shape[0] != k * c_in or tuple(in_grads.shape) != (m, c_out):
        raise RuntimeError(name + ": inconsistent shapes")
    grad_mask = int(grad_mask)
    d_w = torch.empty_like(weights) if grad_mask & GRAD_WEIGHTS else None
    d_f = torch.empty_like(feats) if grad_mask & GRAD_FEATS else None
    d_p = torch.empty_like(pts) if with_pts and grad_mask & GRAD_PTS else None
    d_s = torch.empty_like(samples) if with_pts and grad_mask & GRAD_PTS else None
    proj_p = _conv_proj_arg(name, proj, m, c_in, k, dev)
    ws = _backward_workspace(n, m, t, c_in, k, c_out, grad_mask, dev, mirror)
    _lib.call("pccnn_conv_backward", ctypes.byref(desc), _optr(pts), _ptr(feats), _optr(samples), _ptr(neigh),
              _ptr(ends), _optr(radii), _ptr(weights), _ptr(in_grads), proj_p,
              _mirror_arg(name, mirror, neigh, pts, samples) if with_pts else _P(0), grad_mask, n, m, t, _dims_of(pts), c_in, 1,
              c_out,
              int(divide_by_count), _optr(d_w), _optr(d_f), _optr(d_param_a), _P(0), _optr(d_pdf), _optr(d_p),
              _optr(d_s), _ptr(ws), ws.numel(), _stream())
    return d_w, d_f, d_p, d_s


def _generic_weight_var(name, desc, k, pts, feats, samples, neigh, ends, radii, divide_by_count):
    dev = feats.device
    n, m, t, c_in = feats.shape[0], ends.shape[0], neigh.shape[0], feats.shape[1]
    out = torch.empty((1,), dtype=torch.float32, device=dev)
    ws = _workspace(_lib.load().pccnn_conv_weight_var_workspace_bytes(m, t, c_in, k), dev)
    _lib.call("pccnn_conv_weight_var", ctypes.byref(desc), _optr(pts), _ptr(feats), _optr(samples), _ptr(neigh),
              _ptr(ends), _optr(radii), n, m, t, _dims_of(pts), c_in, int(divide_by_count), _ptr(out), _ptr(ws), ws.numel(),
              _stream())
    return out.reshape(())


def _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts):
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    _chk(pdf, name + ": pdf", torch.float32, 1, dev)
    _chk(kernel_pts, name + ": kernel_pts", torch.float32, 2, dev)
    if pdf.shape[0] != pts.shape[0] or kernel_pts.shape[1] != d:
        raise RuntimeError(name + ": pdf must be [N] and kernel_pts [K, D]")
    return kernel_pts.shape[0]


def kp_conv_n(pts, pdf, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, return_proj=False):
    """kp_conv_n(pts, pdf f32[N], feats, samples, neighbors, start_ids, radii, kernel_pts f32[K,D], sigma,
    weights f32[K*Cin,Cout]) -> f32[M,Cout]: KPConv whose correlation is divided by the density of the neighbor
    (pccnn_lib_ops/pcconvs/kpconvn.cuh:32-42)."""
    name = "kp_conv_n"
    if _is_planar(pts):
        return kp_conv_n(_pad_cols(pts), pdf, feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                         _pad_cols(kernel_pts), sigma, weights, return_proj)
    k = _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts)
    desc = _basis(BASIS_KPN, k, kernel_pts, sigma=sigma, pdf=pdf)
    return _generic_forward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, False, return_proj)


def kp_conv_n_grads(pts, pdf, feats, samples, neigh, ends, radii, kernel_pts, sigma, weights, in_grads, proj=None,
                    grad_mask=GRAD_ALL, mirror=None):
    """kp_conv_n_grads(..., in_grads) -> [dW, dFeat, dKernelPts, dPts, dSamples]; the density gets no gradient
    (pccnn_lib_ops/pcconvs/kpconvn.cuh:57-68)."""
    name = "kp_conv_n_grads"
    if _is_planar(pts):
        g = kp_conv_n_grads(_pad_cols(pts), pdf, feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                            _pad_cols(kernel_pts), sigma, weights, in_grads, proj, grad_mask, mirror)
        return [g[0], g[1], _cut(g[2]), _cut(g[3]), _cut(g[4])]
    k = _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts)
    desc = _basis(BASIS_KPN, k, kernel_pts, sigma=sigma, pdf=pdf)
    d_kp = torch.empty_like(kernel_pts) if int(grad_mask) & GRAD_BASIS_PARAMS else None
    d_w, d_f, d_p, d_s = _generic_backward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, in_grads,
                                           proj, grad_mask, False, d_param_a=d_kp, mirror=mirror)
    return [d_w, d_f, d_kp, d_p, d_s]


def kp_conv_n_weight_var(pts, pdf, feats, samples, neigh, ends, radii, kernel_pts, sigma):
    """kp_conv_n_weight_var(...) -> 0-d float tensor (pccnn_lib_ops/pcconvs/kpconvn.cuh:83-92)."""
    name = "kp_conv_n_weight_var"
    if _is_planar(pts):
        return kp_conv_n_weight_var(_pad_cols(pts), pdf, feats, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                                    _pad_cols(kernel_pts), sigma)
    k = _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts)
    desc = _basis(BASIS_KPN, k, kernel_pts, sigma=sigma, pdf=pdf)
    return _generic_weight_var(name, desc, k, pts, feats, samples, neigh, ends, radii, False)


def pccnn(pts, feats, pdf, samples, neigh, ends, radii, kernel_pts, sigma, weights, return_proj=False):
    """pccnn(pts, feats, pdf f32[N], samples, neighbors, start_ids, radii, kernel_pts f32[K,D], sigma,
    weights f32[K*Cin,Cout]) -> f32[M,Cout]: gaussian kernel-point correlation divided by the density
    (pccnn_lib_ops/pcconvs/pccnn.cuh:32-42; note the feats-before-pdf argument order)."""
    name = "pccnn"
    if _is_planar(pts):
        return pccnn(_pad_cols(pts), feats, pdf, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                     _pad_cols(kernel_pts), sigma, weights, return_proj)
    k = _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts)
    desc = _basis(BASIS_GAUSS, k, kernel_pts, sigma=sigma, pdf=pdf)
    return _generic_forward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, False, return_proj)


def pccnn_grads(pts, feats, pdf, samples, neigh, ends, radii, kernel_pts, sigma, weights, in_grads, proj=None,
                grad_mask=GRAD_ALL, mirror=None):
    """pccnn_grads(..., in_grads) -> [dW, dFeat, dKernelPts, dPdf, dPts, dSamples]
    (pccnn_lib_ops/pcconvs/pccnn.cuh:57-68)."""
    name = "pccnn_grads"
    if _is_planar(pts):
        g = pccnn_grads(_pad_cols(pts), feats, pdf, _pad_cols(samples), neigh, ends, _pad_cols(radii, 1.0),
                        _pad_cols(kernel_pts), sigma, weights, in_grads, proj, grad_mask, mirror)
        return [g[0], g[1], _cut(g[2]), g[3], _cut(g[4]), _cut(g[5])]
    k = _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts)
    desc = _basis(BASIS_GAUSS, k, kernel_pts, sigma=sigma, pdf=pdf)
    d_kp = torch.empty_like(kernel_pts) if int(grad_mask) & GRAD_BASIS_PARAMS else None
    d_pdf = torch.empty_like(pdf) if int(grad_mask) & GRAD_PDF else None
    d_w, d_f, d_p, d_s = _generic_backward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, in_grads,
                                           proj, grad_mask, False, d_param_a=d_kp, d_pdf=d_pdf, mirror=mirror)
    return [d_w, d_f, d_kp, d_pdf, d_p, d_s]


def pccnn_weight_variance(pts, feats, pdf, samples, neigh, ends, radii, kernel_pts, sigma):
    """pccnn_weight_variance(...) -> 0-d float tensor (pccnn_lib_ops/pcconvs/pccnn.cuh:83-92)."""
    name = "pccnn_weight_variance"
    if _is_planar(pts):
        return pccnn_weight_variance(_pad_cols(pts), feats, pdf, _pad_cols(samples), neigh, ends,
                                     _pad_cols(radii, 1.0), _pad_cols(kernel_pts), sigma)
    k = _kernel_pts_args(name, pts, pdf, feats, samples, neigh, ends, radii, kernel_pts)
    desc = _basis(BASIS_GAUSS, k, kernel_pts, sigma=sigma, pdf=pdf)
    return _generic_weight_var(name, desc, k, pts, feats, samples, neigh, ends, radii, False)


def _sph_args(name, pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins):
    d, dev = _conv_args(name, pts, feats, samples, neigh, ends, radii)
    _conv_dims(pts, name, only_3d=True)      # spherical coordinates
    for b, what in ((radial_bins, "radial"), (azimuth_bins, "azimuth"), (polar_bins, "polar")):
        _chk(b, "%s: %s bins" % (name, what), torch.float32, 1, dev)
        if b.shape[0] < 1:
            raise RuntimeError("%s: empty %s bins" % (name, what))
    k = radial_bins.shape[0] * azimuth_bins.shape[0] * polar_bins.shape[0] + 1
    return k, _basis(BASIS_SPH, k, radial_bins, azimuth_bins, polar_bins)


def sph_conv(pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins, weights,
             return_proj=False):
    """sph_conv(pts, feats, samples, neighbors, start_ids, radii, radial_bins f32[R], azimuth_bins f32[A],
    polar_bins f32[P], weights f32[(R*A*P+1)*Cin, Cout]) -> f32[M,Cout]: one-hot spherical-bin correlation, divided
    by the neighbor count (pccnn_lib_ops/pcconvs/sphconv.cuh:19-29)."""
    name = "sph_conv"
    k, desc = _sph_args(name, pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins)
    return _generic_forward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, True, return_proj)


def sph_conv_grads(pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins, weights, in_grads,
                   proj=None, grad_mask=GRAD_WEIGHTS | GRAD_FEATS):
    """sph_conv_grads(..., in_grads) -> [dW, dFeat] (pccnn_lib_ops/pcconvs/sphconv.cuh:31-42)."""
    name = "sph_conv_grads"
    k, desc = _sph_args(name, pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins)
    d_w, d_f, _, _ = _generic_backward(name, desc, k, pts, feats, samples, neigh, ends, radii, weights, in_grads,
                                       proj, int(grad_mask) & (GRAD_WEIGHTS | GRAD_FEATS | GRAD_DETERMINISTIC), True, with_pts=False)
    return [d_w, d_f]


def sph_conv_weight_var(pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins):
    """sph_conv_weight_var(...) -> 0-d float tensor; the per-sample sums are divided by the squared neighbor count
    (pccnn_lib_ops/pcconvs/sphconv.cuh:44-55)."""
    name = "sph_conv_weight_var"
    k, desc = _sph_args(name, pts, feats, samples, neigh, ends, radii, radial_bins, azimuth_bins, polar_bins)
    return _generic_weight_var(name, desc, k, pts, feats, samples, neigh, ends, radii, True)


def _linear_basis_args(name, pts, radii, samples, neigh, axis, bias):
    _chk(pts, name + ": pts", torch.float32, 2)
    dev = pts.device
    d = _conv_dims(pts, name)
    _chk(samples, name + ": samples", torch.float32, 2, dev)
    _chk(neigh, name + ": neighbors", torch.int32, 2, dev)
    _chk(radii, name + ": radii", torch.float32, 1, dev)
    _chk(axis, name + ": axis", torch.float32, 2, dev)
    bias = _chk(bias, name + ": bias", torch.float32, None, dev)
    k = axis.shape[1]
    if samples.shape[1] != d or neigh.shape[1] != 2 or radii.shape[0] != d or axis.shape[0] != d or bias.numel() != k:
        raise RuntimeError(name + ": axis must be [D, K], bias [1, K] or [K], radii [D]")
    return d, dev, k


def point_conv_basis(pts, radii, samples, neigh, axis, bias):
    """point_conv_basis(pts, radii, samples, neighbors, axis f32[D,K], bias f32[1,K]) -> f32[T,K]: the affine map
    of the normalised offsets that PointConv feeds to its own layers (pccnn_lib_ops/pcconvs/pointconv.cuh:20-26)."""
    name = "point_conv_basis"
    if _is_planar(pts):
        return point_conv_basis(_pad_cols(pts), _pad_cols(radii, 1.0), _pad_cols(samples), neigh, _pad_rows(axis), bias)
    d, dev, k = _linear_basis_args(name, pts, radii, samples, neigh, axis, bias)
    t = neigh.shape[0]
    out = torch.empty((t, k), dtype=torch.float32, device=dev)
    _lib.call("pccnn_linear_basis_forward", _ptr(pts), _ptr(samples), _ptr(neigh), _ptr(radii), _ptr(axis),
              _ptr(bias), pts.shape[0], samples.shape[0], t, d, k, _ptr(out), _stream())
    return out


def point_conv_basis_grads(pts, radii, samples, neigh, axis, bias, in_grads):
    """point_conv_basis_grads(..., in_grads f32[T,K]) -> [dPts, dSamples, dAxis, dBias f32[1,K]]
    (pccnn_lib_ops/pcconvs/pointconv.cuh:28-35)."""
    name = "point_conv_basis_grads"
    if _is_planar(pts):
        g = point_conv_basis_grads(_pad_cols(pts), _pad_cols(radii, 1.0), _pad_cols(samples), neigh, _pad_rows(axis),
                                   bias, in_grads)
        return [_cut(g[0]), _cut(g[1]), g[2][:2].contiguous(), g[3]]
    d, dev, k = _linear_basis_args(name, pts, radii, samples, neigh, axis, bias)
    t = neigh.shape[0]
    in_grads = _chk(in_grads.contiguous(), name + ": in_grads", torch.float32, 2, dev)
    if tuple(in_grads.shape) != (t, k):
        raise RuntimeError(name + ": in_grads must be [T, K]")
    d_p, d_s, d_a = torch.empty_like(pts), torch.empty_like(samples), torch.empty_like(axis)
    d_b = torch.empty((1, k), dtype=torch.float32, device=dev)
    ws = _workspace(_lib.load().pccnn_linear_basis_workspace_bytes(t), dev)
    _lib.call("pccnn_linear_basis_backward", _ptr(pts), _ptr(samples), _ptr(neigh), _ptr(radii), _ptr(axis),
              _ptr(bias), _ptr(in_grads), pts.shape[0], samples.shape[0], t, d, k, _ptr(d_p), _ptr(d_s), _ptr(d_a),
              _ptr(d_b), _ptr(ws), ws.numel(), _stream())
    return [d_p, d_s, d_a, d_b]


def _explicit_args(name, basis, feats, neigh, ends):
    _chk(basis, name + ": basis", torch.float32, 2)
    dev = basis.device
    _chk(feats, name + ": features", torch.float32, 2, dev)
    _chk(neigh, name + ": neighbors", torch.int32, 2, dev)
    _chk(ends, name + ": start_ids", torch.int32, 1, dev)
    if basis.shape[0] != neigh.shape[0] or neigh.shape[1] != 2:
        raise RuntimeError(name + ": basis must be [T, K] and neighbors [T, 2]")
    k = basis.shape[1]
    return k, _basis(BASIS_EXPLICIT, k, basis)


def point_conv(basis, feats, neigh, ends, weights, return_proj=False):
    """point_conv(basis f32[T,K], feats, neighbors, start_ids, weights f32[K*Cin,Cout]) -> f32[M,Cout]: the
    correlation with per-pair basis values given by the caller (pccnn_lib_ops/pcconvs/pointconv.cuh:37-42)."""
    name = "point_conv"
    k, desc = _explicit_args(name, basis, feats, neigh, ends)
    return _generic_forward(name, desc, k, None, feats, None, neigh, ends, None, weights, False, return_proj)


def point_conv_grads(basis, feats, neigh, ends, weights, in_grads, proj=None, grad_mask=GRAD_ALL):
    """point_conv_grads(..., in_grads) -> [dW, dFeat, dBasis f32[T,K]] (pccnn_lib_ops/pcconvs/pointconv.cuh:44-50)."""
    name = "point_conv_grads"
    k, desc = _explicit_args(name, basis, feats, neigh, ends)
    d_b = torch.empty_like(basis) if int(grad_mask) & GRAD_BASIS_PARAMS else None
    d_w, d_f, _, _ = _generic_backward(name, desc, k, None, feats, None, neigh, ends, None, weights, in_grads, proj,
                                       int(grad_mask) & (GRAD_WEIGHTS | GRAD_FEATS | GRAD_BASIS_PARAMS | GRAD_DETERMINISTIC), False,
                                       d_param_a=d_b, with_pts=False)
    return [d_w, d_f, d_b]


def point_conv_weight_var(basis, feats, neigh, ends):
    """point_conv_weight_var(basis, feats, neighbors, start_ids) -> 0-d float tensor
    (pccnn_lib_ops/pcconvs/pointconv.cuh:52-56)."""
    name = "point_conv_weight_var"
    k, desc = _explicit_args(name, basis, feats, neigh, ends)
    return _generic_weight_var(name, desc, k, None, feats, None, neigh, ends, None, False)


REFERENCE_NAMES = (
    "build_grid_ds", "compute_keys", "find_neighbors", "compute_pdf", "compute_pdf_grads", "poisson_disk_sampling",
    "mc_conv", "mc_conv_grads", "mc_conv_weight_var", "point_conv_basis", "point_conv_basis_grads", "point_conv",
    "point_conv_grads", "point_conv_weight_var", "kp_conv", "kp_conv_grads", "kp_conv_weight_var", "kp_conv_n",
    "kp_conv_n_grads", "kp_conv_n_weight_var", "sph_conv", "sph_conv_grads", "sph_conv_weight_var", "pccnn",
    "pccnn_grads", "pccnn_weight_variance")


# ----------------------------------------------------------------------------- bindings
#
# Two bindings of the same C ABI serve the 26 reference names: the compiled extension module ``pccnn_lib_ops`` (what
# the reference builds from setup.py:7-31; csrc/ops_module.cpp here: pybind11, TORCH_CHECK contracts, at::empty
# outputs, torch's current HIP stream) and the ctypes functions above, which need no compiler.  The compiled one is
# used when it has been built; ``use_binding`` switches.  Functions beyond the 26 names exist only in this module.

BINDINGS = {"ctypes": {name: globals()[name] for name in REFERENCE_NAMES}}
binding = "ctypes"


def _load_compiled():
    import importlib.util
    import os
    import sys
    mod = sys.modules.get("pccnn_lib_ops")
    if mod is not None and getattr(mod, "binding", None) == "compiled":
        return mod
    from .build import extension_path
    path = extension_path()
    if not os.path.exists(path):
        return None
    _lib.load()                                   # libpccnn_hip.so first, by its path
    spec = importlib.util.spec_from_file_location("pccnn_lib_ops", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    sys.modules.setdefault("pccnn_lib_ops", mod)    # a later ``import pccnn_lib_ops`` gets this very module
    return mod


def use_binding(which):
    """Route the 26 reference names through the "compiled" extension or through "ctypes"; returns the name of the
    binding in use before the call.  Raises if the compiled module has not been built."""
    global binding
    if which not in BINDINGS:
        if which != "compiled":
            raise RuntimeError("use_binding: 'compiled' or 'ctypes', got %r" % (which,))
        mod = _load_compiled()
        if mod is None:
            raise RuntimeError("use_binding: the compiled pccnn_lib_ops extension has not been built "
                               "(python -m pccnn_lib_amd.build)")
        BINDINGS["compiled"] = {name: getattr(mod, name) for name in REFERENCE_NAMES}
    before, binding = binding, which
    globals().update(BINDINGS[which])
    return before


def _initial_binding():
    """The compiled binding when it has been built, unless the environment asks for the other
    (PCCNN_LIB_OPS_BINDING=ctypes|compiled; asking for a compiled module that is not there is an error)."""
    import os
    asked = os.environ.get("PCCNN_LIB_OPS_BINDING", "")
    if asked:
        use_binding(asked)
        return
    try:
        use_binding("compiled")
    except (RuntimeError, ImportError, OSError):      # not built (or built for another torch): ctypes it is
        pass


_initial_binding()
