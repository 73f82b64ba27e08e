"""Operator layer (``equitorch.ops``): table-driven sparse products and the indexed scale-segment reduction,
backed by the HIP kernels of ``libcgtp``."""
from .batched_sparse_dense_op import (
    indexed_inner_scale_gather,
    indexed_mat_t_vec_scale_gather,
    indexed_mul_scale_gather,
    indexed_outer_scale_gather,
    indexed_scavec_scale_gather,
    indexed_vecmat_scale_gather,
    indexed_vecsca_scale_gather,
)
from .indexed_scale_segment_op import indexed_scale_segment
from .spherical_harmonics import spherical_harmonics

__all__ = [
    "indexed_mul_scale_gather", "indexed_vecsca_scale_gather", "indexed_scavec_scale_gather",
    "indexed_inner_scale_gather", "indexed_outer_scale_gather", "indexed_vecmat_scale_gather",
    "indexed_mat_t_vec_scale_gather", "indexed_scale_segment", "spherical_harmonics",
]
