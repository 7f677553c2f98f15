"""Channel-wise tensor product whose second operand is the spherical harmonics of a 3-vector, as one polynomial.

The reference evaluates ``SphericalHarmonics`` (``cuequivariance_torch/operations/spherical_harmonics.py:26-93``, descriptor
``cuequivariance/group_theory/descriptors/spherical_harmonics_.py:23-52``) and hands its output to
``ChannelWiseTensorProduct`` (``cuequivariance_torch/operations/tp_channel_wise.py:30-258``) as the operand ``x2``.  Here the
harmonics are substituted into the product's scalar paths: a path ``(w, x1, x2[j], out)`` with coefficient ``c`` and a term
``coef * v[i1] ... v[il]`` of ``Y_j`` give the path ``(w, x1, v[i1], ..., v[il], out)`` with coefficient ``c * coef`` of the
operation that reads the vector ``l`` times.  The result is an ordinary ``SegmentedPolynomial`` over ``(w, x1, vector) -> out``
- the executors, the backward tables and the oracle take it as it is - and the structure kept beside it lets the generated
edge kernels evaluate the harmonics in registers instead of reading them from memory.
"""

from __future__ import annotations

from collections import defaultdict
from dataclasses import dataclass
from typing import Dict, List, Sequence, Tuple

from . import descriptors
from .irreps import Irreps
from .polynomial import Operation, SegmentedPolynomial
from .stp import SegmentedTensorProduct


@dataclass(frozen=True)
class FusedHarmonics:
    """What ``channelwise_spherical`` substituted: the flattened product (operands ``w[u], x1[u], x2[], out[u]``), the degrees
    and, per component ``j`` of ``x2``, the terms ``(sorted vector indices, coefficient)`` of ``Y_j`` (permutations merged)."""

    product: SegmentedPolynomial
    ls: Tuple[int, ...]
    terms: Tuple[Tuple[Tuple[Tuple[int, ...], float], ...], ...]

    def __hash__(self):
        return hash((self.ls, self.terms))


def harmonics_terms(ir_vec, ls: Sequence[int]) -> List[List[Tuple[Tuple[int, ...], float]]]:
    """Per output component of ``descriptors.spherical_harmonics(ir_vec, ls)``: its monomials as (sorted indices into the
    vector, coefficient), the permutations of one monomial summed."""
    sh = descriptors.spherical_harmonics(ir_vec, list(ls)).polynomial.flatten_coefficient_modes().squeeze_modes()
    ncomp = sh.outputs[0].num_segments
    merged: List[Dict[Tuple[int, ...], float]] = [defaultdict(float) for _ in range(ncomp)]
    for _, stp in sh.operations:
        for path in stp.paths:
            merged[path.indices[-1]][tuple(sorted(path.indices[:-1]))] += float(path.coefficients)
    return [sorted((k, c) for k, c in m.items() if c != 0.0) for m in merged]


def channelwise_spherical(irreps_in1: Irreps, ls: Sequence[int], filter_irreps_out=None):
    """``(polynomial, FusedHarmonics, irreps_out)`` of ``channelwise_tensor_product(irreps_in1, Y_ls, filter)`` with ``Y_ls(vector)``
    substituted for the second operand.  Inputs ``w, x1, vector (3)``, output as for the plain product; rows ``ir_mul``."""
    ls = tuple(ls)
    group = irreps_in1.irrep_class
    ir_vec = group(1, -1) if group.__name__ == "O3" else group(1)
    sh = descriptors.spherical_harmonics(ir_vec, list(ls))
    e = descriptors.channelwise_tensor_product(irreps_in1, sh.outputs[0].irreps, filter_irreps_out)
    product = e.polynomial.flatten_coefficient_modes().squeeze_modes()
    (ope, stp), = product.operations
    assert tuple(ope.buffers) == (0, 1, 2, 3) and str(stp.subscripts) == "u,u,,u", (ope, stp.subscripts)
    w_op, x1_op, x2_op, out_op = stp.operands
    shf = sh.polynomial.flatten_coefficient_modes().squeeze_modes()
    assert shf.outputs[0].num_segments == x2_op.num_segments
    v_op = shf.inputs[0]

    # every ordered index tuple of the harmonics' own paths (their sum is the polynomial; the backward tables differentiate
    # each occurrence of the vector in turn)
    by_component = defaultdict(list)
    for _, sstp in shf.operations:
        for path in sstp.paths:
            by_component[path.indices[-1]].append((tuple(path.indices[:-1]), float(path.coefficients)))
    by_degree: Dict[int, Dict[tuple, float]] = defaultdict(lambda: defaultdict(float))
    for path in stp.paths:
        ws, x1s, j, outs = path.indices
        for vi, coef in by_component[j]:
            by_degree[len(vi)][(ws, x1s, *vi, outs)] += float(path.coefficients) * coef
    operations = []
    for degree, paths in sorted(by_degree.items()):
        d = SegmentedTensorProduct.from_subscripts("u,u" + "," * degree + ",u")
        d.add_segments(0, w_op.segments)
        d.add_segments(1, x1_op.segments)
        for t in range(degree):
            d.add_segments(2 + t, v_op.segments)
        d.add_segments(2 + degree, out_op.segments)
        for idx, c in sorted(paths.items()):
            if c != 0.0:
                d.add_path(*idx, c=c)
        operations.append((Operation((0, 1) + (2,) * degree + (3,)), d))
    poly = SegmentedPolynomial([w_op, x1_op, v_op], [out_op], operations)
    info = FusedHarmonics(product, ls, tuple(tuple(t) for t in harmonics_terms(ir_vec, ls)))
    return poly, info, e.outputs[0].irreps
