"""Text point-cloud loader and normaliser (CPU only)."""
import numpy as np
import pytest

from pccnn_lib_amd import xyz


def test_load_and_normalize_round_trip(tmp_path):
    rng = np.random.default_rng(0)
    pts = rng.uniform(-30, 40, (500, 3))
    path = tmp_path / "model.xyz"
    np.savetxt(path, pts, fmt="%.6f")
    got = xyz.load_xyz(str(path))
    assert got.shape == (500, 3) and np.allclose(got, np.loadtxt(path), rtol=0, atol=0)
    norm = xyz.normalize_to_unit_diagonal(got)
    assert norm.dtype == np.float32
    # the box is centred on the origin and its diagonal has length one (unit_test/unit_test.py:46-51)
    assert np.allclose(norm.max(axis=0) + norm.min(axis=0), 0, atol=1e-6)
    assert np.isclose(np.linalg.norm(norm.max(axis=0) - norm.min(axis=0)), 1.0, atol=1e-6)
    # similarity transform: distance ratios are preserved
    d0 = np.linalg.norm(got[0] - got[1]) / np.linalg.norm(got[2] - got[3])
    d1 = np.linalg.norm(norm[0].astype(np.float64) - norm[1]) / np.linalg.norm(norm[2].astype(np.float64) - norm[3])
    assert np.isclose(d0, d1, rtol=1e-4)


def test_extra_columns_batch_and_errors(tmp_path):
    rng = np.random.default_rng(1)
    a, b = rng.normal(size=(40, 6)), rng.normal(size=(30, 3))
    pa, pb = tmp_path / "a.xyz", tmp_path / "b.xyz"
    np.savetxt(pa, a)
    np.savetxt(pb, b)
    assert np.allclose(xyz.load_xyz(str(pa)), a[:, :3])
    pts, ids = xyz.load_batch([str(pa), str(pb)], 25)
    assert pts.shape == (50, 3) and pts.dtype == np.float32 and ids.dtype == np.int32
    assert list(np.bincount(ids)) == [25, 25]
    bad = tmp_path / "bad.xyz"
    bad.write_text("1 2\n3 4\n")
    with pytest.raises(RuntimeError, match="three columns"):
        xyz.load_xyz(str(bad))
    ragged = tmp_path / "ragged.xyz"
    ragged.write_text("1 2 3\n4 5\n")
    with pytest.raises(RuntimeError, match="ragged"):
        xyz.load_xyz(str(ragged))
