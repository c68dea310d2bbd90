"""Hand-worked known answers for poisson_disk_sampling, written from the reference's rule
(pccnn_lib_ops/poisson_disk_sampling/poisson_disk_sampling.cu:56-105, :158-192) and from nothing else:

  * 2^D launches, launch c = 0 .. 2^D - 1 in ascending order; launch c visits the cells whose
    coordinate in dimension i has parity (c >> i) & 1, dimension 0 in the LOWEST bit (:165-170, :66-72);
  * inside a cell the points are visited in ascending sorted index (:82-84);
  * a point is selected iff none of its listed neighbors is selected yet (:91-104).

Every case is a list of points given as (cell coordinates incl. cloud, neighbors by name); the expected
selection is derived by hand in the comments.  Keys follow grid_utils.cuh:85-93:
key = ((b * nc0 + c0) * nc1 + c1) * nc2 + c2.  The ids below are sorted indices (points listed in key order).
"""
import numpy as np


def _pack(num_cells, points, links):
    """points: list of (name, cloud, cell tuple) ALREADY in ascending key order; links: undirected pairs of
    names.  Returns (sorted_keys i64[N], neigh i32[T,2] (point, sample), ends i32[N], num_cells i32[D])."""
    names = [p[0] for p in points]
    keys = []
    for _, b, cell in points:
        k = b
        for c, n in zip(cell, num_cells):
            k = k * n + c
        keys.append(k)
    assert keys == sorted(keys), "list the points in key order"
    adj = {n: {n} for n in names}          # every point neighbors itself
    for a, b in links:
        adj[a].add(b)
        adj[b].add(a)
    neigh, ends = [], []
    for s, n in enumerate(names):
        for m in sorted(names.index(x) for x in adj[n]):
            neigh.append((m, s))
        ends.append(len(neigh))
    return (np.asarray(keys, np.int64), np.asarray(neigh, np.int32).reshape(-1, 2), np.asarray(ends, np.int32),
            np.asarray(num_cells, np.int32))


def case_3d():
    """Grid 3 x 2 x 4, three clouds (24 keys per cloud).

    cloud 0: b in cell (0,1,0) [key 4, parity (0,1,0) -> launch 2], a in cell (1,0,0) [key 8, parity (1,0,0)
             -> launch 1]; a ~ b.  Launch 1 runs before launch 2: a is selected, b then sees a and is rejected.
             (Descending launches, dimension 0 in the highest bit, or plain sorted order would all select b.)
    cloud 1: c in (0,0,0) [key 24, launch 0], e in (1,1,1) [key 37, launch 7], d in (2,1,2) [key 46, parity
             (0,1,0) -> launch 2]; c ~ e, d ~ e.  Launch 0 selects c, launch 2 selects d (e is not selected
             yet), launch 7 rejects e.  (Descending launches select only e; so does descending launches
             combined with the reversed bit order.)
    cloud 2: f, g, h in cell (1,1,2) [key 62, parity (1,1,0) -> launch 3], i in (1,1,3) [key 63, launch 7];
             f ~ g, g ~ h, h ~ i.  Inside the cell in sorted order: f selected, g rejected (f), h selected (g is
             not selected); launch 7: i rejected (h).
    Sorted indices: b0 a1 c2 e3 d4 f5 g6 h7 i8  ->  selected {1, 2, 4, 5, 7}."""
    pts = [("b", 0, (0, 1, 0)), ("a", 0, (1, 0, 0)),
           ("c", 1, (0, 0, 0)), ("e", 1, (1, 1, 1)), ("d", 1, (2, 1, 2)),
           ("f", 2, (1, 1, 2)), ("g", 2, (1, 1, 2)), ("h", 2, (1, 1, 2)), ("i", 2, (1, 1, 3))]
    links = [("a", "b"), ("c", "e"), ("d", "e"), ("f", "g"), ("g", "h"), ("h", "i")]
    return _pack((3, 2, 4), pts, links), np.asarray([1, 2, 4, 5, 7], np.int64)


def case_2d():
    """Grid 2 x 3, one cloud.  b in (0,1) [key 1, parity (0,1) -> launch 2], c in (0,2) [key 2, launch 0],
    a in (1,0) [key 3, parity (1,0) -> launch 1], d in (1,1) [key 4, launch 3]; a ~ b, c ~ d.  Launch 0 selects c,
    launch 1 selects a, launch 2 rejects b (a), launch 3 rejects d (c).
    Sorted indices b0 c1 a2 d3 -> selected {1, 2}."""
    pts = [("b", 0, (0, 1)), ("c", 0, (0, 2)), ("a", 0, (1, 0)), ("d", 0, (1, 1))]
    links = [("a", "b"), ("c", "d")]
    return _pack((2, 3), pts, links), np.asarray([1, 2], np.int64)


def case_4d():
    """Grid 2 x 2 x 2 x 2, one cloud: z in (0,0,0,0) [key 0, launch 0], x in (0,0,0,1) [key 1, launch 8],
    y in (1,0,0,0) [key 8, launch 1], w in (1,1,1,1) [key 15, launch 15]; x ~ y, z ~ w.  Launch 0 selects z,
    launch 1 selects y, launch 8 rejects x (y), launch 15 rejects w (z).
    Sorted indices z0 x1 y2 w3 -> selected {0, 2}."""
    pts = [("z", 0, (0, 0, 0, 0)), ("x", 0, (0, 0, 0, 1)), ("y", 0, (1, 0, 0, 0)), ("w", 0, (1, 1, 1, 1))]
    return _pack((2, 2, 2, 2), pts, [("x", "y"), ("z", "w")]), np.asarray([0, 2], np.int64)


CASES = {"3d": case_3d, "2d": case_2d, "4d": case_4d}
