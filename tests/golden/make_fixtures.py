"""Regenerates tests/golden/models_4x1024.npy from the reference's own test data.

The reference's unit tests load 32 text point clouds (unit_test/point_clouds/model*.xyz,
100 000 rows of "x y z") and normalise each by its bounding-box centre and diagonal
(unit_test/unit_test.py:43-51).  This script applies the same normalisation to the first
four files and keeps the first 1024 rows of each as float32: a small data fixture
(inputs only).  It runs in the build container only (the reference tree is not present on
the GPU machine); the tests read the committed .npy file.
"""
import os
import sys

import numpy as np

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    out = np.zeros((4, 1024, 3), np.float32)
    for i in range(4):
        model = np.loadtxt(os.path.join(REF, "unit_test", "point_clouds", "model%d.xyz" % i))
        mx, mn = model.max(axis=0), model.min(axis=0)
        center = (mx + mn) * 0.5
        size = np.linalg.norm(mx - mn)
        out[i] = ((model - center) / size).astype(np.float32)[:1024]
    np.save(os.path.join(HERE, "models_4x1024.npy"), out)
    print("wrote", out.shape, out.dtype)


if __name__ == "__main__":
    main()
