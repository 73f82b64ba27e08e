"""Module layer (``equitorch.nn``) of the sparse tensor-product path."""
from . import functional
from .activations import Gate
from .cutoffs import CosineCutoff, MollifierCutoff, PolynomialCutoff
from .linears import IrrepsLinear, IrrepWiseLinear, SO3Linear
from .norm import MeanSquaredNorm, Norm, SquaredNorm
from .normalization import BatchRMSNorm, LayerRMSNorm
from .radials import BesselBasis
from .sphericals import SphericalHarmonics, SphericalToXYZ, XYZToSpherical
from .tensor_products import TensorProduct

__all__ = ["SO3Linear", "IrrepsLinear", "IrrepWiseLinear", "TensorProduct", "SphericalHarmonics", "XYZToSpherical", "SphericalToXYZ", "Gate", "SquaredNorm", "Norm", "MeanSquaredNorm",
           "BatchRMSNorm", "LayerRMSNorm", "BesselBasis", "PolynomialCutoff", "CosineCutoff", "MollifierCutoff",
           "functional"]
