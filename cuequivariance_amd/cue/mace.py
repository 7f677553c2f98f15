"""Symmetric contraction in the parametrisation of the original MACE implementation.

``symmetric_contraction(irreps_in, irreps_out, degrees)`` returns the standard descriptor
(:func:`cuequivariance_amd.cue.descriptors.symmetric_contraction`) together with a projection
matrix ``p`` of shape ``(num_mace_weights, num_weights)``: weights ``w_mace[a, u]`` trained with
the original MACE basis act like ``w[b, u] = sum_a w_mace[a, u] p[a, b]`` in the standard one.

Restates ``cuequivariance/group_theory/experimental/mace/symmetric_contractions.py:27-265`` of the
reference (the generalised Wigner coupling ``:202-265`` follows MACE's ``tools/cg.py``).
"""

from __future__ import annotations

import functools
from typing import Optional

import numpy as np

from .descriptors import _symmetric_contraction_core
from .irreps import Irrep, Irreps, IrrepsAndLayout, clebsch_gordan, ir_mul
from .linalg import round_to_sqrt_rational, triu_array
from .polynomial import EquivariantPolynomial, Operation, SegmentedPolynomial
from .stp import SegmentedTensorProduct


def symmetric_contraction(irreps_in: Irreps, irreps_out: Irreps, degrees):
    """``(EquivariantPolynomial, projection)``; operands ``weights[u], input[u] -> output[u]``."""
    poly, projection = _cached(irreps_in, irreps_out, tuple(degrees))
    e = EquivariantPolynomial(
        [IrrepsAndLayout(irreps_in.new_scalars(poly.inputs[0].size), ir_mul), IrrepsAndLayout(irreps_in, ir_mul)],
        [IrrepsAndLayout(irreps_out, ir_mul)],
        poly,
    )
    return e, projection


def _dense_coefficients(d: SegmentedTensorProduct) -> np.ndarray:
    m = np.zeros([ope.num_segments for ope in d.operands])
    for path in d.paths:
        m[tuple(path.indices)] = path.coefficients
    return m


@functools.lru_cache(maxsize=None)
def _cached(irreps_in: Irreps, irreps_out: Irreps, degrees: tuple):
    assert min(degrees) > 0
    # the original MACE layout of weights: per output irrep, degrees descending
    mace_poly = SegmentedPolynomial.stack(
        [
            SegmentedPolynomial.stack(
                [_mace_poly(irreps_in, irreps_out[i: i + 1], n) for n in reversed(degrees)], [True, False, False]
            )
            for i in range(len(irreps_out))
        ],
        [True, False, True],
    )
    std_poly = _symmetric_contraction_core(irreps_in, irreps_out, tuple(degrees))
    mats = []
    for pol in (mace_poly, std_poly):
        cols = []
        for _, d in pol.operations:
            m = _dense_coefficients(d.symmetrize_operands(range(1, d.num_operands - 1)))
            cols.append(m.reshape(m.shape[0], -1))
        mats.append(np.concatenate(cols, axis=1))
    a1, a2 = mats
    used = np.nonzero(np.any(a1 != 0, axis=0) | np.any(a2 != 0, axis=0))[0]  # lighter pseudo-inverse
    a1, a2 = a1[:, used], a2[:, used]
    projection = round_to_sqrt_rational(a1 @ np.linalg.pinv(a2))
    np.testing.assert_allclose(a1, projection @ a2, atol=1e-7)
    return std_poly, projection


def _mace_poly(irreps_in: Irreps, irreps_out: Irreps, degree: int) -> SegmentedPolynomial:
    mul = irreps_in.muls[0]
    assert all(m == mul for m in irreps_in.muls) and all(m == mul for m in irreps_out.muls)
    irreps_in, irreps_out = irreps_in.set_mul(1), irreps_out.set_mul(1)
    abc = "abcdefgh"[:degree]
    d = SegmentedTensorProduct.from_subscripts(f"u_{'_'.join(abc)}_i+{abc}ui")
    for i in range(1, degree + 1):
        d.add_segment(i, (irreps_in.dim,))
    for _, ir in irreps_out:
        u = np.moveaxis(U_matrix_real(irreps_in, ir, degree), 0, -1)  # (d_in, ..., d_in, solutions, ir.dim)
        if u.shape[-2] == 0:
            d.add_segment(degree + 1, {"i": ir.dim})
        else:
            d.add_path(None, *(0,) * degree, None, c=triu_array(u, degree))
    d = d.flatten_coefficient_modes()
    d = d.append_modes_to_all_operands("u", {"u": mul})
    assert d.num_operands >= 3
    return SegmentedPolynomial(
        [d.operands[0], d.operands[1]], [d.operands[-1]], [(Operation([0] + [1] * degree + [2]), d)]
    )


def U_matrix_real(irreps_in: Irreps, ir_out: Irrep, correlation: int) -> np.ndarray:
    """All couplings of ``correlation`` copies of ``irreps_in`` onto ``ir_out``:
    shape ``(ir_out.dim, d_in, ..., d_in, num_solutions)``."""
    G = type(ir_out)
    mid = frozenset(G(l, (-1) ** l) for l in range(12)) if correlation == 4 else None
    arrays = [base for ir, base in _wigner_nj(irreps_in, correlation, mid) if ir == ir_out]
    if arrays:
        return np.stack(arrays, axis=-1)
    return np.zeros((ir_out.dim,) + (irreps_in.dim,) * correlation + (0,))


@functools.lru_cache(maxsize=None)
def _wigner_nj(irreps_in: Irreps, degree: int, filter_ir_mid: Optional[frozenset]):
    """Left-to-right coupling tree: list of ``(irrep, tensor of shape (irrep.dim, d_in, ..., d_in))``."""
    assert degree > 0
    if degree == 1:
        out, eye, off = [], np.eye(irreps_in.dim), 0
        for mul, ir in irreps_in:
            for _ in range(mul):
                out.append((ir, eye[off: off + ir.dim]))
                off += ir.dim
        return out
    out = []
    for ir_left, C_left in _wigner_nj(irreps_in, degree - 1, filter_ir_mid):
        off = 0
        for mul, ir in irreps_in:
            for ir_out in ir_left * ir:
                if filter_ir_mid is not None and ir_out not in filter_ir_mid:
                    continue
                for cg in clebsch_gordan(ir_left, ir, ir_out):
                    C = np.einsum("jk,jli->ikl", C_left.reshape(ir_left.dim, -1), cg)
                    C = np.reshape(C, (ir_out.dim,) + (irreps_in.dim,) * (degree - 1) + (ir.dim,))
                    C = round_to_sqrt_rational(C)
                    for u in range(mul):
                        E = np.zeros((ir_out.dim,) + (irreps_in.dim,) * degree)
                        E[..., off + u * ir.dim: off + (u + 1) * ir.dim] = C
                        out.append((ir_out, E))
            off += mul * ir.dim
    return sorted(out, key=lambda t: t[0])
