"""Text point-cloud ingestion: the ``x y z`` files and the normalisation the reference's test driver applies
before anything reaches the GPU (unit_test/unit_test.py:43-51)."""
import numpy as np


def load_xyz(p_path, p_max_points=None):
    """Reads a whitespace-separated text file of ``x y z [more columns]`` rows -> float64 [N, 3]."""
    with open(p_path, "r") as handle:
        first = handle.readline().split()
        if len(first) < 3:
            raise RuntimeError("%s: expected at least three columns, got %d" % (p_path, len(first)))
        handle.seek(0)
        flat = np.array(handle.read().split(), dtype=np.float64)
    if flat.size % len(first) != 0:
        raise RuntimeError("%s: ragged rows (%d values, %d columns)" % (p_path, flat.size, len(first)))
    pts = flat.reshape(-1, len(first))[:, :3]
    return pts if p_max_points is None else pts[:p_max_points]


def normalize_to_unit_diagonal(p_pts):
    """Centres a cloud on the middle of its bounding box and divides by the length of the box diagonal, so the
    cloud fits a ball of diameter one (unit_test/unit_test.py:46-51).  Returns float32."""
    pts = np.asarray(p_pts, dtype=np.float64)
    max_pt, min_pt = pts.max(axis=0), pts.min(axis=0)
    center = (max_pt + min_pt) * 0.5
    aabb_size = np.linalg.norm(max_pt - min_pt)
    return ((pts - center) / aabb_size).astype(np.float32)


def load_batch(p_paths, p_points_per_cloud=None):
    """Loads and normalises several files -> (pts float32 [N, 3], batch_ids int32 [N])."""
    clouds = [normalize_to_unit_diagonal(load_xyz(path))[:p_points_per_cloud] for path in p_paths]
    ids = [np.full(cloud.shape[0], i, np.int32) for i, cloud in enumerate(clouds)]
    return np.ascontiguousarray(np.concatenate(clouds, axis=0)), np.concatenate(ids)
