"""Functional layer (``equitorch.nn.functional``) of the sparse tensor-product path."""
from .activations import gating
from .angular import sincos
from .cutoffs import cosine_cutoff, mollifier_cutoff, polynomial_cutoff, radial_standarize
from .dropout import irrep_wise_dropout
from .rotations import angles_to_matrix
from .edge import (EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_radial,
                   edge_tensor_product_uu_vectors)
from .linears import (irrep_wise_linear, irreps_linear, so2_linear_uu, so2_linear_uv, so3_linear_uu, so3_linear_uv, tensor_product_1uu, tensor_product_1vu, tensor_product_u1u,
                      tensor_product_u1v, tensor_product_uu1, tensor_product_vu1)
from .norm import batch_mean_squared_norm, channel_mean_squared_norm, norm, squared_norm
from .normalization import batch_rms_norm, layer_rms_norm
from .sparse_product import (sparse_inner, sparse_mat_t_vec, sparse_mul, sparse_outer, sparse_scavec, sparse_vecmat,
                             sparse_vecsca)
from .sparse_scale import sparse_scale
from .sphericals import spherical_harmonics, spherical_to_xyz, xyz_to_sincos, xyz_to_spherical
from .wigner_d import align_to_z_wigner_d, dense_wigner_rotation, sparse_wigner_rotation, wigner_d_matrix
from .tensor_products import tensor_dot_uu, tensor_dot_uv, tensor_product_uuu, tensor_product_uvw

__all__ = [
    "tensor_product_uuu", "tensor_product_uvw", "tensor_product_u1u", "tensor_product_1uu", "tensor_product_uu1",
    "tensor_product_u1v", "tensor_product_1vu", "tensor_product_vu1", "so3_linear_uu", "so3_linear_uv", "irreps_linear", "irrep_wise_linear",
    "sparse_mul", "sparse_outer", "sparse_inner", "sparse_vecmat", "sparse_vecsca", "sparse_scavec",
    "sparse_mat_t_vec", "sparse_scale", "EdgePlan", "edge_tensor_product_uu", "edge_tensor_product_uu_vectors", "edge_tensor_product_uu_radial", "spherical_harmonics",
    "xyz_to_spherical", "spherical_to_xyz", "gating", "squared_norm", "norm", "channel_mean_squared_norm",
    "batch_mean_squared_norm", "batch_rms_norm", "layer_rms_norm", "radial_standarize", "polynomial_cutoff",
    "cosine_cutoff", "mollifier_cutoff", "sincos", "xyz_to_sincos", "sparse_wigner_rotation",
    "dense_wigner_rotation", "wigner_d_matrix", "align_to_z_wigner_d", "irrep_wise_dropout", "angles_to_matrix", "so2_linear_uu", "so2_linear_uv", "tensor_dot_uu", "tensor_dot_uv",
]
