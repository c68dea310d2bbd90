"""Host-side helpers for preparing point clouds (pccnn_lib/py_utils/__init__.py:1): numpy only, as in the reference."""
from .augmentation import (anisotropic_scale_pc, farthest_point_sampling, jitter_pc, mirror_pc, poisson_disk_sampling,
                           rotate_pc_3d, uniform_samples_sphere, uniform_samples_surface_sphere)

__all__ = ["jitter_pc", "mirror_pc", "anisotropic_scale_pc", "rotate_pc_3d", "uniform_samples_surface_sphere",
           "uniform_samples_sphere", "poisson_disk_sampling", "farthest_point_sampling"]
