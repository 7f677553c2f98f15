"""Torch-facing layer: the drop-in mirror of ``cuequivariance_torch`` running on HIP kernels."""

from .transpose import TransposeSegments, TransposeIrrepsLayout
from .segmented_polynomial import SegmentedPolynomial
from .operations import (ChannelWiseSphericalTensorProduct, ChannelWiseTensorProduct, FullyConnectedTensorProduct, Linear, SymmetricContraction,
                         SphericalHarmonics, Rotation, Inversion, encode_rotation_angle, vector_to_euler_angles)
from .uniform_1d import uniform_1d
from .deprecated import TensorProduct, EquivariantTensorProduct, SymmetricTensorProduct, IWeightedSymmetricTensorProduct
from .triangle import triangle_multiplicative_update, TriMulPrecision
from . import layers
from . import dense as _dense  # noqa: F401  (defines the operators dense_fwd / dense_bwd that saved graphs of Linear and the fully connected product call)

__all__ = [
    "TransposeSegments",
    "TransposeIrrepsLayout",
    "SegmentedPolynomial",
    "ChannelWiseSphericalTensorProduct",
    "ChannelWiseTensorProduct",
    "FullyConnectedTensorProduct",
    "Linear",
    "SymmetricContraction",
    "SphericalHarmonics",
    "Rotation",
    "Inversion",
    "encode_rotation_angle",
    "vector_to_euler_angles",
    "uniform_1d",
    "TensorProduct",
    "EquivariantTensorProduct",
    "SymmetricTensorProduct",
    "IWeightedSymmetricTensorProduct",
    "triangle_multiplicative_update",
    "TriMulPrecision",
    "layers",
]
