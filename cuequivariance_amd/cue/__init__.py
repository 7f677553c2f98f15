"""Descriptor side: irreps, Clebsch-Gordan coefficients, segmented tensor products and polynomials."""

from .irreps import (
    Irrep,
    SU2,
    SO3,
    O3,
    MulIrrep,
    Irreps,
    IrrepsLayout,
    mul_ir,
    ir_mul,
    IrrepsAndLayout,
    clebsch_gordan,
    into_list_of_irrep,
)
from .stp import Subscripts, SegmentedOperand, Path, SegmentedTensorProduct
from .polynomial import Operation, SegmentedPolynomial, EquivariantPolynomial
from . import descriptors

__all__ = [
    "Irrep", "SU2", "SO3", "O3", "MulIrrep", "Irreps", "IrrepsLayout", "mul_ir", "ir_mul",
    "IrrepsAndLayout", "clebsch_gordan", "into_list_of_irrep", "Subscripts", "SegmentedOperand",
    "Path", "SegmentedTensorProduct", "Operation", "SegmentedPolynomial", "EquivariantPolynomial",
    "descriptors",
]
