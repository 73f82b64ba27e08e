"""Table builders and index helpers (the tensor-product subset of ``equitorch.utils``)."""
from ._indices import expand_left, extract_batch_segments, extract_scatter_indices, sort_by_column_key
from ._random import rand_rotation_angles, rand_rotation_matrices, rand_spherical_angles, rand_spherical_xyz
from ._structs import (
    create_irreps_linear_info,
    create_tp_info,
    generate_fully_connected_irreps_linear_paths,
    generate_fully_connected_tp_paths,
    irreps_blocks_infos,
    irreps_info,
    j_matrix_info,
    so2_linear_info,
    so2_linear_infos,
    wigner_d_info,
    z_rotation_infos,
    irreps_linear_infos,
    prepare_irreps_linear,
    prepare_so3,
    sparse_product_info,
    sparse_product_infos,
    sparse_scale_info,
    sparse_scale_infos,
    tp_infos,
)

__all__ = [
    "rand_spherical_xyz", "expand_left", "extract_batch_segments", "sort_by_column_key",
    "extract_scatter_indices", "sparse_scale_info", "sparse_scale_infos", "sparse_product_info",
    "sparse_product_infos", "generate_fully_connected_tp_paths", "tp_infos",
    "generate_fully_connected_irreps_linear_paths", "irreps_linear_infos", "irreps_info", "z_rotation_infos", "j_matrix_info", "wigner_d_info", "so2_linear_infos",
    "so2_linear_info", "irreps_blocks_infos", "rand_spherical_angles", "rand_rotation_angles", "rand_rotation_matrices",
]
