"""Descriptor side: irreps, Clebsch-Gordan coefficients, segmented tensor products and polynomials."""

from .irreps import (
    Irrep,
    SU2,
    SO3,
    O3,
    O3_e3nn,
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
from .reduced_basis import (
    IrrepsArray,
    reduced_tensor_product_basis,
    reduced_symmetric_tensor_product_basis,
    reduced_antisymmetric_tensor_product_basis,
    selection_rule_product,
    selection_rule_power,
)
from .irreps import assume, get_irrep_scope, get_layout_scope
from . import descriptors
from . import mace
from . import segmented_polynomials
from . import group_theory

__version__ = "0.1.0"

__all__ = [
    "Irrep", "SU2", "SO3", "O3", "O3_e3nn", "MulIrrep", "Irreps", "IrrepsLayout", "mul_ir", "ir_mul",
    "IrrepsAndLayout", "clebsch_gordan", "into_list_of_irrep", "Subscripts", "SegmentedOperand",
    "Path", "SegmentedTensorProduct", "Operation", "SegmentedPolynomial", "EquivariantPolynomial",
    "descriptors", "mace", "IrrepsArray", "reduced_tensor_product_basis", "reduced_symmetric_tensor_product_basis",
    "reduced_antisymmetric_tensor_product_basis", "selection_rule_product", "selection_rule_power",
    "assume", "get_irrep_scope", "get_layout_scope", "__version__", "segmented_polynomials", "group_theory",
]
