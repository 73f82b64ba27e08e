"""Module layer (``equitorch.nn``) of the sparse tensor-product path."""
from . import functional
from .activations import Gate
from .angular import SinCos
from .dropout import Dropout
from .others import Separable, SplitIrreps
from .rotations import AnglesToMatrix
from .cutoffs import CosineCutoff, MollifierCutoff, PolynomialCutoff
from .linears import IrrepsLinear, IrrepWiseLinear, SO2Linear, SO3Linear
from .norm import MeanSquaredNorm, Norm, SquaredNorm
from .normalization import BatchRMSNorm, LayerRMSNorm
from .radials import BesselBasis
from .init import initialize_linear, initialize_so3_so2_linear, initialize_tensor_product
from .sphericals import SphericalHarmonics, SphericalToXYZ, XYZToSinCos, XYZToSpherical
from .tensor_products import TensorDot, TensorProduct
from .wigner_d import AlignToZWignerD, DenseWignerRotation, SparseWignerRotation, WignerD

__all__ = ["SO3Linear", "IrrepsLinear", "IrrepWiseLinear", "TensorProduct", "SphericalHarmonics", "XYZToSpherical", "SphericalToXYZ", "Gate", "SquaredNorm", "Norm", "MeanSquaredNorm",
           "BatchRMSNorm", "LayerRMSNorm", "BesselBasis", "PolynomialCutoff", "CosineCutoff", "MollifierCutoff",
           "SO2Linear", "SinCos", "SparseWignerRotation", "DenseWignerRotation", "WignerD", "AlignToZWignerD",
           "Dropout", "SplitIrreps", "Separable", "AnglesToMatrix", "TensorDot", "XYZToSinCos", "initialize_tensor_product",
           "initialize_so3_so2_linear", "initialize_linear", "functional"]
