"""Functional layer (``equitorch.nn.functional``) of the sparse tensor-product path."""
from .edge import EdgePlan, edge_tensor_product_uu
from .linears import so3_linear_uu, tensor_product_1uu, tensor_product_u1u, tensor_product_uu1
from .sparse_product import sparse_inner, sparse_mul, sparse_scavec, sparse_vecsca
from .sparse_scale import sparse_scale
from .tensor_products import tensor_product_uuu

__all__ = [
    "tensor_product_uuu", "tensor_product_u1u", "tensor_product_1uu", "tensor_product_uu1", "so3_linear_uu",
    "sparse_mul", "sparse_inner", "sparse_vecsca", "sparse_scavec", "sparse_scale",
    "EdgePlan", "edge_tensor_product_uu",
]
