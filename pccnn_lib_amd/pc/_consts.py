"""Small per-dimension constants (radii, bandwidths, cell sizes) as device tensors.

The reference turns such an argument into a tensor on every call (``torch.as_tensor(p_radius, device=...)``,
pccnn_lib/pc/layers/IConvLayer.py:129-131, pc/Pointcloud.py:89-91, pc/Grid.py:23).  From host memory that is a
synchronous copy: the host waits until the device has finished everything queued before, which for a small level of
a hierarchy costs more than the level's kernels.  A value that was seen before is therefore served from a table of
the tensors already on the device; tensors that are on the device already pass through untouched."""
import numbers

import numpy as np
import torch

_table = {}
_host_values = {}        # id(tensor of the table) -> (the tensor, the host values it was made from)
_MAX_ENTRIES = 256


def device_vector(value, num_dims, device):
    """``value`` (number, sequence, numpy array or tensor) as a float32 tensor of ``num_dims`` entries on ``device``;
    a scalar is repeated.  Treat the result as read-only: equal values share one tensor."""
    if torch.is_tensor(value):
        out = value.to(device=device, dtype=torch.float32)
        return out.repeat(num_dims) if out.dim() == 0 else out
    if isinstance(value, numbers.Real):
        flat = (float(value),) * num_dims
    else:
        arr = np.asarray(value, dtype=np.float32).reshape(-1)
        flat = tuple(float(v) for v in arr) if arr.size > 1 else (float(arr[0]),) * num_dims
    key = (flat, str(device))
    out = _table.get(key)
    if out is None:
        if len(_table) >= _MAX_ENTRIES:
            _table.clear()
            _host_values.clear()
        out = torch.tensor(flat, dtype=torch.float32, device=device)
        _table[key] = out
        _host_values[id(out)] = (out, np.asarray(flat, dtype=np.float32))
    return out


def host_vector(tensor):
    """The host values (float32 numpy array) behind a tensor that ``device_vector`` made from host data, or None for
    any other tensor: lets a caller do on the host, with the same fp32 arithmetic, what would otherwise need a
    read-back.  A table tensor that somebody wrote to in place (its version counter moved) no longer counts: the
    kernels would read the new values while the host sized grids from the old ones."""
    entry = _host_values.get(id(tensor)) if tensor is not None else None
    if entry is None or entry[0] is not tensor or tensor._version != 0:
        return None
    return entry[1]


def host_num_cells(box_host, cell_host):
    """Grid size as a list of ints from the box and the cell size on the host: the fp32 arithmetic of
    pccnn_lib/pc/Grid.py:26-28 (subtract, IEEE divide, truncate, + 1, maximum over the clouds) in numpy."""
    mn, mx = box_host
    with np.errstate(all="ignore"):
        cells = ((mx - mn) / cell_host.reshape(1, -1)).astype(np.int32) + np.int32(1)
    return [int(v) for v in cells.max(axis=0)]
