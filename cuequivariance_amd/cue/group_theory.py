"""The names of the reference's ``cuequivariance.group_theory`` package that exist here (irreps, layouts, Clebsch-Gordan
coefficients, reduced bases, equivariant polynomials, descriptors)."""

from . import descriptors
from .irreps import (SO3, SU2, O3, Irrep, Irreps, IrrepsAndLayout, IrrepsLayout, MulIrrep, assume, clebsch_gordan, get_irrep_scope,
                     get_layout_scope, ir_mul, mul_ir)
from .polynomial import EquivariantPolynomial
from .reduced_basis import (reduced_antisymmetric_tensor_product_basis, reduced_symmetric_tensor_product_basis,
                            reduced_tensor_product_basis, selection_rule_power, selection_rule_product)

__all__ = ["Irrep", "clebsch_gordan", "selection_rule_product", "selection_rule_power", "SU2", "SO3", "O3", "get_irrep_scope",
           "MulIrrep", "Irreps", "IrrepsLayout", "mul_ir", "ir_mul", "IrrepsAndLayout", "get_layout_scope", "assume",
           "reduced_tensor_product_basis", "reduced_symmetric_tensor_product_basis", "reduced_antisymmetric_tensor_product_basis",
           "EquivariantPolynomial", "descriptors"]
