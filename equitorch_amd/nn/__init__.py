"""Module layer (``equitorch.nn``) of the sparse tensor-product path."""
from . import functional
from .linears import IrrepsLinear, IrrepWiseLinear, SO3Linear
from .sphericals import SphericalHarmonics, SphericalToXYZ, XYZToSpherical
from .tensor_products import TensorProduct

__all__ = ["SO3Linear", "IrrepsLinear", "IrrepWiseLinear", "TensorProduct", "SphericalHarmonics", "XYZToSpherical", "SphericalToXYZ", "functional"]
