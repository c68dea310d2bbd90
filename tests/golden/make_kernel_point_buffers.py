"""Regenerates tests/golden/kernel_point_buffers.npz: the ``kernel_pts_`` / ``sigma_`` buffers a freshly built
reference KPConv layer holds, for each of the reference's twelve constant kernel-point layouts.

The constant tables are read as TEXT from the reference's data file
(pccnn_lib/pc/layers/kernel_points/kernel_points.py:3-364; number literals are parsed, nothing is imported or
executed), then the steps of pccnn_lib/pc/layers/KPConv.py:46-57 are applied with plain numpy: float32 norms,
division by the largest norm, smallest non-centre norm d, (3-D only) the rotation that rotate_pc_3d
(pccnn_lib/py_utils/pc_utils.py:94-125) builds from RandomState(15), float32 rounding, division by 1 + d;
sigma = d / (1 + d).  It runs in the build container only (the reference tree is not present on the GPU machine);
the tests read the committed .npz file.
"""
import os
import re
import sys

import numpy as np

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def read_tables():
    text = open(os.path.join(REF, "pccnn_lib", "pc", "layers", "kernel_points", "kernel_points.py")).read()
    tables = {}
    for m in re.finditer(r"'(\d+)_(\d+)'\s*:\s*np\.array\(\[(.*?)\]\)", text, re.S):
        rows = [[float(v) for v in r.split(",")] for r in re.findall(r"\[([^\[\]]+)\]", m.group(3))]
        tables[m.group(1) + "_" + m.group(2)] = np.array(rows)
    return tables


def layer_buffers(table):
    pts = table.astype(np.float32)
    norms = np.linalg.norm(pts, axis=-1).astype(np.float32)
    largest = np.amax(norms)
    norms = norms / largest
    pts = pts / largest
    d = np.amin(norms[1:])
    if pts.shape[-1] == 3:
        a = (np.random.RandomState(15).random_sample((3)) - 0.5) * 2.0 * (2.0 * np.pi)
        c, s = np.cos(a), np.sin(a)
        about_x = np.array([[1.0, 0.0, 0.0], [0.0, c[0], -s[0]], [0.0, s[0], c[0]]])
        about_y = np.array([[c[1], 0.0, s[1]], [0.0, 1.0, 0.0], [-s[1], 0.0, c[1]]])
        about_z = np.array([[c[2], -s[2], 0.0], [s[2], c[2], 0.0], [0.0, 0.0, 1.0]])
        pts = np.dot(pts, np.dot(about_z, np.dot(about_y, about_x)))
    pts = pts.astype(np.float32)
    return pts / (1.0 + d), np.float32((d * 1.0) / (1.0 + d))


def main():
    out = {}
    for key, table in sorted(read_tables().items()):
        out["table_" + key] = table
        out["kernel_pts_" + key], out["sigma_" + key] = layer_buffers(table)
    assert len(out) == 36, len(out)
    np.savez(os.path.join(HERE, "kernel_point_buffers.npz"), **out)
    print("wrote", len(out) // 3, "layouts")


if __name__ == "__main__":
    main()
