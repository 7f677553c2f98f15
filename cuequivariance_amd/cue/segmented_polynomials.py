"""The names of the reference's ``cuequivariance.segmented_polynomials`` package that exist here, and ``dot``.

``dot(x, y, (i, j))`` composes two segmented tensor products over a common operand (reference
``cuequivariance/segmented_polynomials/dot.py:37-109``): read as multilinear maps, operand ``i`` of ``x`` and operand ``j`` of
``y`` - the same segments under the same subscripts - are summed over, the other operands of ``x`` and then of ``y`` remain.
Every pair of paths that meet in a segment of the contracted operand gives one path whose coefficients are the product of the
two (``einsum`` over the union of the coefficient subscripts); with no pair given the result is the plain product.
"""

from __future__ import annotations

import itertools

import numpy as np

from .polynomial import Operation, SegmentedPolynomial
from .stp import Path, SegmentedOperand, SegmentedTensorProduct, Subscripts

__all__ = ["Subscripts", "Path", "SegmentedOperand", "SegmentedTensorProduct", "Operation", "SegmentedPolynomial", "dot",
           "compute_last_operand"]


def _unique(text: str) -> str:
    return "".join(dict.fromkeys(text))


def dot(x: SegmentedTensorProduct, y: SegmentedTensorProduct, *contraction) -> SegmentedTensorProduct:
    for i, j in contraction:
        if x.operands_and_subscripts[i] != y.operands_and_subscripts[j]:
            raise ValueError("Operands to contract must be the same.")
    keep_x = [k for k in range(x.num_operands) if all(k != i for i, _ in contraction)]
    keep_y = [k for k in range(y.num_operands) if all(k != j for _, j in contraction)]
    coeff = _unique(x.coefficient_subscripts + y.coefficient_subscripts)
    d = SegmentedTensorProduct([x.operands_and_subscripts[k] for k in keep_x] + [y.operands_and_subscripts[k] for k in keep_y], coeff)
    formula = f"{x.coefficient_subscripts},{y.coefficient_subscripts}->{coeff}"
    by_segments = {}
    for py in y.paths:  # the paths of y by the segments they take of the contracted operands
        by_segments.setdefault(tuple(py.indices[j] for _, j in contraction), []).append(py)
    for px in x.paths:
        for py in by_segments.get(tuple(px.indices[i] for i, _ in contraction), []) if contraction else y.paths:
            d.add_path(*[px.indices[k] for k in keep_x], *[py.indices[k] for k in keep_y],
                       c=np.einsum(formula, px.coefficients, py.coefficients))
    return d


def compute_last_operand(d: SegmentedTensorProduct, *inputs: np.ndarray, dtype=None) -> np.ndarray:
    """The last operand of ``d`` from the others, in numpy (reference ``segmented_polynomials/evaluate.py:25-139``)."""
    return d.compute_last_operand(*inputs, dtype=dtype)
