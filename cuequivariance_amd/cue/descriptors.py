"""Ready-made equivariant polynomials: channel-wise / fully-connected tensor products, linear maps.

Reference behaviour followed (``cuequivariance/cuequivariance/group_theory/descriptors``):

* ``irreps_tp.py:22-91``    fully_connected_tensor_product  ``"uvw,iu,jv,kw+ijk"``
* ``irreps_tp.py:232-321``  channelwise_tensor_product      ``"uv,iu,jv,kuv+ijk"``
* ``irreps_tp.py:505-545``  linear                          ``"uv,iu,iv"``
* ``irreps_tp.py:127-195``  full_tensor_product             ``"iu,jv,kuv+ijk"`` (the channel-wise product without weights)
* ``irreps_tp.py:364-461``  elementwise_tensor_product      ``"iu,ju,ku+ijk"`` (equal channels multiplied, multiplicities aligned)
* ``transposition.py:18-36``  transpose                     ``"ui,iu"`` / ``"iu,ui"`` between the two layouts
* ``spherical_harmonics_.py:23-85,119-156`` spherical-harmonics polynomial, recursion and normalisation
* ``symmetric_contractions.py:20-134``  symmetric_contraction  ``"w_a_b_c_i+abciw"`` per degree
* ``rotations.py:23-252``  rotations about fixed axes with the angle given as ``[cos(l t) .. cos(t), 1, sin(t) .. sin(l t)]``,
  their compositions ``xy``, ``yx``, ``yxy``, a rotation by a known angle about a known axis, and the inversion

All descriptors use the ``ir_mul`` layout (component index outside, multiplicity inside).
"""

from __future__ import annotations

import functools
import itertools
from typing import Optional, Sequence

import numpy as np

from .irreps import Irrep, Irreps, IrrepsAndLayout, clebsch_gordan, into_list_of_irrep, ir_mul
from .polynomial import EquivariantPolynomial, Operation, SegmentedPolynomial
from .reduced_basis import reduced_symmetric_tensor_product_basis
from .stp import SegmentedOperand, SegmentedTensorProduct

__all__ = [
    "channelwise_tensor_product",
    "fully_connected_tensor_product",
    "linear",
    "full_tensor_product",
    "elementwise_tensor_product",
    "transpose",
    "spherical_harmonics",
    "spherical_harmonics_values",
    "symmetric_contraction",
    "fixed_axis_angle_rotation",
    "x_rotation",
    "y_rotation",
    "xy_rotation",
    "yx_rotation",
    "yxy_rotation",
    "inversion",
]


def _scalar_weights(irreps: Irreps, poly: SegmentedPolynomial) -> IrrepsAndLayout:
    return IrrepsAndLayout(irreps.new_scalars(poly.inputs[0].size), ir_mul)


def channelwise_tensor_product(
    irreps1: Irreps,
    irreps2: Irreps,
    irreps3_filter=None,
    simplify_irreps3: bool = False,
) -> EquivariantPolynomial:
    """``weights[uv], lhs[iu], rhs[jv] -> output[kuv]``: one weighted path per allowed (ir1, ir2, ir3).

    Every path owns a weight segment and an output segment.  Output irreps are
    stable-sorted with the group's order and the weight/output segments are
    renumbered accordingly while the paths keep their generation order.
    """
    G = irreps1.irrep_class
    if irreps3_filter is not None:
        irreps3_filter = into_list_of_irrep(G, irreps3_filter)

    d = SegmentedTensorProduct.from_subscripts("uv,iu,jv,kuv+ijk")
    for mul, ir in irreps1:
        d.add_segment(1, (ir.dim, mul))
    for mul, ir in irreps2:
        d.add_segment(2, (ir.dim, mul))

    out = []
    for (i1, (mul1, ir1)), (i2, (mul2, ir2)) in itertools.product(enumerate(irreps1), enumerate(irreps2)):
        for ir3 in ir1 * ir2:
            if irreps3_filter is not None and ir3 not in irreps3_filter:
                continue
            for cg in clebsch_gordan(ir1, ir2, ir3):
                d.add_path(None, i1, i2, None, c=cg, dims={"u": mul1, "v": mul2})
                out.append((mul1 * mul2, ir3))

    irreps3, _perm, inv = Irreps(G, out).sort()
    d = d.permute_segments(0, inv)
    d = d.permute_segments(3, inv)
    d = d.normalize_paths_for_operand(-1)

    if simplify_irreps3:
        d = d.flatten_coefficient_modes()
        segs = [(ir, k) for _m, ir in irreps3 for k in range(ir.dim)]
        order = sorted(range(len(segs)), key=lambda s: (_Key(segs[s][0]), segs[s][1], s))
        d = d.permute_segments(3, order)
        irreps3 = irreps3.simplify()

    poly = SegmentedPolynomial.eval_last_operand(d)
    return EquivariantPolynomial(
        [_scalar_weights(irreps1, poly), IrrepsAndLayout(irreps1, ir_mul), IrrepsAndLayout(irreps2, ir_mul)],
        [IrrepsAndLayout(irreps3, ir_mul)],
        poly,
    )


class _Key:
    __slots__ = ("ir",)

    def __init__(self, ir):
        self.ir = ir

    def __eq__(self, o):
        return self.ir == o.ir

    def __lt__(self, o):
        return self.ir < o.ir


def fully_connected_tensor_product(irreps1: Irreps, irreps2: Irreps, irreps3: Irreps) -> EquivariantPolynomial:
    """``weights[uvw], lhs[iu], rhs[jv] -> output[kw]``: every allowed (ir1, ir2, ir3) triple gets a weight block."""
    d = SegmentedTensorProduct.from_subscripts("uvw,iu,jv,kw+ijk")
    for mul, ir in irreps1:
        d.add_segment(1, (ir.dim, mul))
    for mul, ir in irreps2:
        d.add_segment(2, (ir.dim, mul))
    for mul, ir in irreps3:
        d.add_segment(3, (ir.dim, mul))
    for (i1, (mul1, ir1)), (i2, (mul2, ir2)), (i3, (mul3, ir3)) in itertools.product(
        enumerate(irreps1), enumerate(irreps2), enumerate(irreps3)
    ):
        if ir3 not in ir1 * ir2:
            continue
        for cg in clebsch_gordan(ir1, ir2, ir3):
            d.add_path((mul1, mul2, mul3), i1, i2, i3, c=cg)
    d = d.normalize_paths_for_operand(-1)
    poly = SegmentedPolynomial.eval_last_operand(d)
    return EquivariantPolynomial(
        [_scalar_weights(irreps1, poly), IrrepsAndLayout(irreps1, ir_mul), IrrepsAndLayout(irreps2, ir_mul)],
        [IrrepsAndLayout(irreps3, ir_mul)],
        poly,
    )


def linear(irreps_in: Irreps, irreps_out: Irreps) -> EquivariantPolynomial:
    """``weights[uv], input[iu] -> output[iv]``: a weight matrix between every pair of equal irreps."""
    d = SegmentedTensorProduct.from_subscripts("uv_iu_iv")
    for mul, ir in irreps_in:
        d.add_segment(1, (ir.dim, mul))
    for mul, ir in irreps_out:
        d.add_segment(2, (ir.dim, mul))
    for (i1, (mul1, ir1)), (i2, (mul2, ir2)) in itertools.product(enumerate(irreps_in), enumerate(irreps_out)):
        if ir1 == ir2:
            d.add_path((mul1, mul2), i1, i2, c=1.0)
    d = d.normalize_paths_for_operand(-1)
    poly = SegmentedPolynomial.eval_last_operand(d)
    return EquivariantPolynomial(
        [_scalar_weights(irreps_in, poly), IrrepsAndLayout(irreps_in, ir_mul)],
        [IrrepsAndLayout(irreps_out, ir_mul)],
        poly,
    )


def full_tensor_product(irreps1: Irreps, irreps2: Irreps, irreps3_filter=None) -> EquivariantPolynomial:
    """``lhs[iu], rhs[jv] -> output[kuv]``: the channel-wise product without weights - every pair of channels of every allowed
    (ir1, ir2, ir3) gets an output channel.  Output irreps stable-sorted like those of the channel-wise product."""
    G = irreps1.irrep_class
    if irreps3_filter is not None:
        irreps3_filter = into_list_of_irrep(G, irreps3_filter)
    d = SegmentedTensorProduct.from_subscripts("iu,jv,kuv+ijk")
    for mul, ir in irreps1:
        d.add_segment(0, (ir.dim, mul))
    for mul, ir in irreps2:
        d.add_segment(1, (ir.dim, mul))
    out = []
    for (i1, (mul1, ir1)), (i2, (mul2, ir2)) in itertools.product(enumerate(irreps1), enumerate(irreps2)):
        for ir3 in ir1 * ir2:
            if irreps3_filter is not None and ir3 not in irreps3_filter:
                continue
            for cg in clebsch_gordan(ir1, ir2, ir3):
                d.add_path(i1, i2, None, c=cg)
                out.append((mul1 * mul2, ir3))
    irreps3, _perm, inv = Irreps(G, out).sort()
    d = d.permute_segments(2, inv).normalize_paths_for_operand(-1)
    return EquivariantPolynomial(
        [IrrepsAndLayout(irreps1, ir_mul), IrrepsAndLayout(irreps2, ir_mul)], [IrrepsAndLayout(irreps3, ir_mul)],
        SegmentedPolynomial.eval_last_operand(d))


def _cut_to_common_multiplicities(irreps1: Irreps, irreps2: Irreps):
    """Both lists of (multiplicity, irrep) cut so that entry k of one has the multiplicity of entry k of the other: the longer
    entry is split into the common part and the rest, which meets the next entry of the other list.  In ``ir_mul`` rows a split
    keeps the memory order only for irreps of dimension one."""
    if irreps1.num_irreps != irreps2.num_irreps:
        raise ValueError(f"The input irreps must have the same number of irreps, got {irreps1} and {irreps2}")
    a, b = [(m, ir) for m, ir in irreps1], [(m, ir) for m, ir in irreps2]
    k = 0
    while k < min(len(a), len(b)):
        (m1, ir1), (m2, ir2) = a[k], b[k]
        if m1 < m2:
            assert ir2.dim == 1, "splitting the channels of an irrep of dimension above one does not keep ir_mul rows in order"
            b[k:k + 1] = [(m1, ir2), (m2 - m1, ir2)]
        elif m2 < m1:
            assert ir1.dim == 1, "splitting the channels of an irrep of dimension above one does not keep ir_mul rows in order"
            a[k:k + 1] = [(m2, ir1), (m1 - m2, ir1)]
        k += 1
    assert [m for m, _ in a] == [m for m, _ in b], (a, b)
    return Irreps(irreps1.irrep_class, a), Irreps(irreps2.irrep_class, b)


def elementwise_tensor_product(irreps1: Irreps, irreps2: Irreps, irreps3_filter=None) -> EquivariantPolynomial:
    """``lhs[iu], rhs[ju] -> output[ku]``: channel n of the first operand with channel n of the second (the operands must hold
    the same number of irreps; multiplicities are aligned by cutting).  The output keeps the order of the products."""
    G = irreps1.irrep_class
    if irreps3_filter is not None:
        irreps3_filter = into_list_of_irrep(G, irreps3_filter)
    cut1, cut2 = _cut_to_common_multiplicities(irreps1, irreps2)
    d = SegmentedTensorProduct.from_subscripts("iu,ju,ku+ijk")
    out = []
    for (mul, ir1), (_, ir2) in zip(cut1, cut2):
        i1, i2 = d.add_segment(0, (ir1.dim, mul)), d.add_segment(1, (ir2.dim, mul))
        for ir3 in ir1 * ir2:
            if irreps3_filter is not None and ir3 not in irreps3_filter:
                continue
            for cg in clebsch_gordan(ir1, ir2, ir3):
                d.add_path(i1, i2, None, c=cg)
                out.append((mul, ir3))
    d = d.normalize_paths_for_operand(-1)
    return EquivariantPolynomial(
        [IrrepsAndLayout(cut1, ir_mul), IrrepsAndLayout(cut2, ir_mul)], [IrrepsAndLayout(Irreps(G, out), ir_mul)],
        SegmentedPolynomial.eval_last_operand(d))


def transpose(irreps: Irreps, source, target) -> EquivariantPolynomial:
    """``input -> output``: the same features in the other layout (``mul_ir``: component inside, ``ir_mul``: channel inside); one
    path of coefficient one per irrep."""
    from .irreps import mul_ir

    d = SegmentedTensorProduct.from_subscripts(("ui" if source == mul_ir else "iu") + "," + ("ui" if target == mul_ir else "iu"))
    for mul, ir in irreps:
        d.add_path(None, None, c=1.0, dims={"u": mul, "i": ir.dim})
    return EquivariantPolynomial([IrrepsAndLayout(irreps, source)], [IrrepsAndLayout(irreps, target)],
                                 SegmentedPolynomial.eval_last_operand(d))


def spherical_harmonics_values(ir_vec: Irrep, ls: Sequence[int], vectors: np.ndarray) -> np.ndarray:
    """Component-normalised real spherical harmonics ``Y_l(x)`` as homogeneous polynomials of ``x``.

    ``Y_0 = 1``, ``Y_1 = sqrt(3) x``, ``Y_l = sqrt(2l+1) CG(Y_l1, Y_l2) / norm`` with ``l1 = l - l//2``,
    ``l2 = l//2`` and ``norm`` fixed by evaluating at ``(0, 1, 0)``.  On unit vectors
    ``sum_m Y_lm^2 = 2l+1``.  Output: ``(..., sum(2l+1))`` in the order of ``ls``.
    """
    vectors = np.asarray(vectors, dtype=np.float64)
    assert vectors.shape[-1] == 3
    return np.concatenate([_normalised_sh(ir_vec, ell, vectors) for ell in ls], axis=-1)


def _normalised_sh(ir_vec: Irrep, ell: int, x: np.ndarray) -> np.ndarray:
    if ell == 0:
        return np.ones(x.shape[:-1] + (1,))
    if ell == 1:
        return np.sqrt(3.0) * x
    l2 = ell // 2
    l1 = ell - l2
    north = np.array([0.0, 1.0, 0.0])

    def raw(v):
        y1, y2 = _normalised_sh(ir_vec, l1, v), _normalised_sh(ir_vec, l2, v)
        ir1 = _sh_irrep(ir_vec, l1)
        ir2 = _sh_irrep(ir_vec, l2)
        ir = sorted(ir1 * ir2, key=_Key)[-1]
        cg = clebsch_gordan(ir1, ir2, ir)[0]
        return np.einsum("...i,...j,ijk->...k", y1, y2, cg)

    norm = np.sqrt(np.sum(raw(north) ** 2))
    return np.sqrt(2 * ell + 1) * raw(x) / norm


def _sh_irrep(ir_vec: Irrep, ell: int) -> Irrep:
    if ell == 0:
        return ir_vec.trivial()
    if ell == 1:
        return ir_vec
    l2 = ell // 2
    l1 = ell - l2
    return sorted(_sh_irrep(ir_vec, l1) * _sh_irrep(ir_vec, l2), key=_Key)[-1]


# ---------------------------------------------------------------------------------------------
# symmetric contraction
# ---------------------------------------------------------------------------------------------
@functools.lru_cache(maxsize=None)
def _symmetric_contraction_core(irreps_in: Irreps, irreps_out: Irreps, degrees: tuple) -> SegmentedPolynomial:
    """Polynomial ``weights[u], x[u] -> out[u]``: for every degree n the symmetric part of ``x^n`` is mapped
    onto ``irreps_out`` with one weight per independent coupling (reference
    ``descriptors/symmetric_contractions.py:20-88``)."""
    degrees = list(degrees)
    if len(degrees) != 1:
        return SegmentedPolynomial.stack(
            [_symmetric_contraction_core(irreps_in, irreps_out, (n,)) for n in degrees], [True, False, False]
        )
    [degree] = degrees
    mul = irreps_in.muls[0]
    assert all(m == mul for m in irreps_in.muls) and all(m == mul for m in irreps_out.muls)
    irreps_in, irreps_out = irreps_in.set_mul(1), irreps_out.set_mul(1)
    x_operands = range(1, degree + 1)
    out_operand = degree + 1
    x_operand = SegmentedOperand([(mul,)] * irreps_in.dim, ndim=1)

    if degree == 0:
        d = SegmentedTensorProduct.from_subscripts("i_i")
        for _, ir in irreps_out:
            if not ir.is_scalar():
                d.add_segment(out_operand, {"i": ir.dim})
            else:
                d.add_path(None, None, c=1, dims={"i": ir.dim})
        d = d.flatten_modes("i")
    else:
        abc = "abcdefgh"[:degree]
        d = SegmentedTensorProduct.from_subscripts(f"w_{'_'.join(abc)}_i+{abc}iw")
        for i in x_operands:
            d.add_segment(i, (irreps_in.dim,))
        U = reduced_symmetric_tensor_product_basis(irreps_in, degree, keep_ir=irreps_out, layout=ir_mul)
        for _, ir in irreps_out:
            u = U.filter(keep=[ir])
            if len(u.segments) == 0:
                d.add_segment(out_operand, {"i": ir.dim})
            else:
                [u] = u.segments  # (a, b, c, ..., i, w)
                d.add_path(None, *(0,) * degree, None, c=u)
        d = d.normalize_paths_for_operand(out_operand)
        d = d.flatten_coefficient_modes()

    d = d.append_modes_to_all_operands("u", {"u": mul})
    for i in x_operands:
        assert d.operands[i] == x_operand
    return SegmentedPolynomial(
        [d.operands[0], x_operand], [d.operands[-1]], [(Operation([0] + [1] * degree + [2]), d)]
    )


def symmetric_contraction(irreps_in: Irreps, irreps_out: Irreps, degrees) -> EquivariantPolynomial:
    """Weighted sum of the input contracted with itself ``degree`` times, for every degree in ``degrees``.

    Operands: ``weights[u], input[u] -> output[u]`` (all ``ir_mul``); the multiplicities of ``irreps_in`` and
    ``irreps_out`` must all be equal and are carried as the parallel mode ``u``.  For ``16x(0+1+2) -> 16x(0+1)`` of SO3
    and degrees (1, 2, 3): 32 + 80 + 176 weights and 4 / 37 / 437 paths (reference
    ``descriptors/symmetric_contractions.py:91-134``)."""
    poly = _symmetric_contraction_core(irreps_in, irreps_out, tuple(degrees))
    return EquivariantPolynomial(
        [IrrepsAndLayout(irreps_in.new_scalars(poly.inputs[0].size), ir_mul), IrrepsAndLayout(irreps_in, ir_mul)],
        [IrrepsAndLayout(irreps_out, ir_mul)],
        poly,
    )


# ---------------------------------------------------------------------------------------------
# spherical harmonics as a polynomial of the vector
# ---------------------------------------------------------------------------------------------
@functools.lru_cache(maxsize=None)
def _sh_monomials(ir_vec: Irrep, ell: int) -> tuple:
    """``Y_l`` component by component as ``{(d0, d1, d2): coefficient}`` (homogeneous of degree ``l``); same
    recursion and normalisation as :func:`spherical_harmonics_values`, carried out on polynomials."""
    from .linalg import round_to_sqrt_rational

    if ell == 0:
        return ({(0, 0, 0): 1.0},)
    if ell == 1:
        return tuple({tuple(int(a == i) for a in range(3)): float(np.sqrt(3.0))} for i in range(3))
    l2 = ell // 2
    l1 = ell - l2
    y1, y2 = _sh_monomials(ir_vec, l1), _sh_monomials(ir_vec, l2)
    ir1, ir2 = _sh_irrep(ir_vec, l1), _sh_irrep(ir_vec, l2)
    ir = sorted(ir1 * ir2, key=_Key)[-1]
    cg = clebsch_gordan(ir1, ir2, ir)[0]
    comps = []
    for k in range(ir.dim):
        acc: dict = {}
        for i in range(ir1.dim):
            for j in range(ir2.dim):
                c = cg[i, j, k]
                if c == 0.0:
                    continue
                for da, ca in y1[i].items():
                    for db, cb in y2[j].items():
                        key = (da[0] + db[0], da[1] + db[1], da[2] + db[2])
                        acc[key] = acc.get(key, 0.0) + c * ca * cb
        comps.append(acc)
    # normalise on the point (0, 1, 0): only the pure x1^l monomials survive there
    north = np.array([comp.get((0, ell, 0), 0.0) for comp in comps])
    scale = np.sqrt(2 * ell + 1) / np.sqrt(np.sum(north**2))
    out = []
    for comp in comps:
        cleaned = {}
        for key, c in comp.items():
            c = float(round_to_sqrt_rational(np.asarray(c * scale), 2**20))
            if abs(c) > 1e-12:
                cleaned[key] = c
        out.append(cleaned)
    return tuple(out)


@functools.lru_cache(maxsize=None)
def _spherical_harmonics_core(ir_vec: Irrep, ls: tuple):
    if len(ls) != 1:
        results = [_spherical_harmonics_core(ir_vec, (ell,)) for ell in ls]
        poly = SegmentedPolynomial.stack([r[0] for r in results], [False, True])
        return poly, Irreps(type(ir_vec), sum([list(r[1]) for r in results], []))
    [ell] = ls
    ir = _sh_irrep(ir_vec, ell)
    assert ir_vec.dim == 3
    d = SegmentedTensorProduct.empty_segments([3] * ell + [ir.dim])
    for i, comp in enumerate(_sh_monomials(ir_vec, ell)):
        for degrees in sorted(comp, reverse=True):  # lexicographic, highest power of x0 first
            indices = sum(((a,) * n for a, n in enumerate(degrees)), ())
            d.add_path(*indices, i, c=comp[degrees])
    d = d.symmetrize_operands(range(ell))
    poly = SegmentedPolynomial(
        [SegmentedOperand([()] * 3, ndim=0)], [SegmentedOperand([()] * ir.dim, ndim=0)], [(Operation([0] * ell + [1]), d)]
    )
    return poly, Irreps(type(ir_vec), [(1, ir)])


def spherical_harmonics(ir_vec: Irrep, ls, layout=ir_mul) -> EquivariantPolynomial:
    """Spherical harmonics ``Y_l(x)`` for every ``l`` in ``ls`` as a polynomial of the vector ``x`` (component
    normalisation: ``sum_m Y_lm(x)^2 = 2l+1`` on unit vectors, ``Y_1 = sqrt(3) x``).  Operands ``vector[] ... -> Y[]``;
    ``[0, 1, 2]`` gives 1 / 3 / 11 paths (reference ``descriptors/spherical_harmonics_.py:56-85``)."""
    poly, irreps_out = _spherical_harmonics_core(ir_vec, tuple(ls))
    return EquivariantPolynomial(
        [IrrepsAndLayout(Irreps(type(ir_vec), [(1, ir_vec)]), ir_mul)], [IrrepsAndLayout(irreps_out, ir_mul)], poly
    )


# ---- rotations and the inversion -------------------------------------------------------------------------------------
# A rotation by the angle t about a coordinate axis acts on an irrep of degree l through D(t) = expm(t X_axis), whose entries
# are linear combinations of cos(m t), sin(m t), m <= l.  The descriptors take the angle as the vector
#   encoding(t) = [cos(L t), cos((L - 1) t), ..., cos(t), 1, sin(t), ..., sin(L t)],   L = lmax,
# so D(t) = sum_e encoding(t)[e] C[e]: the constant matrices C[e] are read off D at sampled angles (a linear system with the
# 2 L + 1 functions as unknowns per entry - exact, the entries lie in their span), not typed in per degree.  Rotations are
# active and right-handed on the components (x, y, z) of a vector: about x by t takes y towards z, about y takes z towards x.


def _rotation_generators(ir: Irrep) -> np.ndarray:
    if type(ir).__name__ not in ("SO3", "O3", "O3_e3nn"):
        raise ValueError(f"Unsupported irrep class {type(ir).__name__}. Must be SO3 or O3.")
    return np.asarray(ir.continuous_generators(), dtype=np.float64)


def _expm(a: np.ndarray) -> np.ndarray:
    from scipy.linalg import expm

    return expm(a)


@functools.lru_cache(maxsize=None)
def _axis_rotation_tensor(ir: Irrep, axis: int, lmax: int) -> np.ndarray:
    """``C[e, j, k]`` with ``D(t)[k, j] = sum_e encoding(t)[e] C[e, j, k]`` for the rotation about coordinate axis ``axis``."""
    if ir.l > lmax:
        raise ValueError(f"lmax = {lmax} is below the degree of {ir}")
    X = _rotation_generators(ir)[axis]
    ts = np.linspace(0.0, 2.0 * np.pi, 4 * lmax + 5, endpoint=False) + 0.1234
    m = np.arange(1, lmax + 1)
    enc = np.concatenate([np.cos(ts[:, None] * m[::-1]), np.ones((len(ts), 1)), np.sin(ts[:, None] * m)], axis=1)
    D = np.stack([_expm(t * X) for t in ts])  # (samples, k, j)
    sol, *_ = np.linalg.lstsq(enc, D.reshape(len(ts), -1), rcond=None)
    assert np.abs(enc @ sol - D.reshape(len(ts), -1)).max() < 1e-10
    C = sol.reshape(2 * lmax + 1, ir.dim, ir.dim).transpose(0, 2, 1)  # (e, j, k)
    C[np.abs(C) < 1e-12] = 0.0
    return C


def _lmax_of(irreps: Irreps, lmax: Optional[int]) -> int:
    for _, ir in irreps:
        _rotation_generators(ir)
    return max(ir.l for _, ir in irreps) if lmax is None else int(lmax)


def _rotation_polynomial(irreps: Irreps, tensors, num_angles: int, lmax: int) -> EquivariantPolynomial:
    """``angle encodings (num_angles of them), input[u] -> output[u]`` with the constant tensor ``tensors(ir)[e1, .., j, k]`` per
    irrep: every encoding component is a scalar segment, every component of an irrep a segment of its multiplicity."""
    d = SegmentedTensorProduct.from_subscripts(",".join([""] * num_angles + ["u", "u"]))
    for a in range(num_angles):
        for _ in range(2 * lmax + 1):
            d.add_segment(a, ())
    for mul, ir in irreps:
        first = d.operands[num_angles].num_segments
        for _ in range(ir.dim):
            d.add_segment(num_angles, (mul,))
            d.add_segment(num_angles + 1, (mul,))
        T = tensors(ir)
        for idx in zip(*np.nonzero(T)):
            *es, j, k = (int(v) for v in idx)
            d.add_path(*es, first + j, first + k, c=float(T[idx]))
    enc = [IrrepsAndLayout(irreps.new_scalars(2 * lmax + 1), ir_mul) for _ in range(num_angles)]
    return EquivariantPolynomial(enc + [IrrepsAndLayout(irreps, ir_mul)], [IrrepsAndLayout(irreps, ir_mul)],
                                 SegmentedPolynomial.eval_last_operand(d))


def _clean(T: np.ndarray) -> np.ndarray:
    T = T.copy()
    T[np.abs(T) < 1e-12] = 0.0
    return T


def y_rotation(irreps: Irreps, lmax: Optional[int] = None) -> EquivariantPolynomial:
    """``phi[], input[u] -> output[u]``: rotation about the y axis, the angle as ``encoding(phi)`` (reference ``rotations.py:131-199``)."""
    L = _lmax_of(irreps, lmax)
    return _rotation_polynomial(irreps, lambda ir: _axis_rotation_tensor(ir, 1, L), 1, L)


def x_rotation(irreps: Irreps, lmax: Optional[int] = None) -> EquivariantPolynomial:
    """``phi[], input[u] -> output[u]``: rotation about the x axis (reference ``rotations.py:202-232``)."""
    L = _lmax_of(irreps, lmax)
    return _rotation_polynomial(irreps, lambda ir: _axis_rotation_tensor(ir, 0, L), 1, L)


def xy_rotation(irreps: Irreps, lmax: Optional[int] = None) -> EquivariantPolynomial:
    """``gamma[], beta[], input[u] -> output[u]``: about y by gamma, then about x by beta (reference ``rotations.py:87-107``)."""
    L = _lmax_of(irreps, lmax)
    return _rotation_polynomial(
        irreps, lambda ir: _clean(np.einsum("cja,bak->cbjk", _axis_rotation_tensor(ir, 1, L), _axis_rotation_tensor(ir, 0, L))), 2, L)


def yx_rotation(irreps: Irreps, lmax: Optional[int] = None) -> EquivariantPolynomial:
    """``phi[], theta[], input[u] -> output[u]``: about x by phi, then about y by theta (reference ``rotations.py:110-128``)."""
    L = _lmax_of(irreps, lmax)
    return _rotation_polynomial(
        irreps, lambda ir: _clean(np.einsum("cja,bak->cbjk", _axis_rotation_tensor(ir, 0, L), _axis_rotation_tensor(ir, 1, L))), 2, L)


def yxy_rotation(irreps: Irreps, lmax: Optional[int] = None) -> EquivariantPolynomial:
    """``gamma[], beta[], alpha[], input[u] -> output[u]``: about y by gamma, then about x by beta, then about y by alpha
    (reference ``rotations.py:49-84``)."""
    L = _lmax_of(irreps, lmax)

    def tensor(ir):
        Y, X = _axis_rotation_tensor(ir, 1, L), _axis_rotation_tensor(ir, 0, L)
        return _clean(np.einsum("cja,bad,edk->cbejk", Y, X, Y))

    return _rotation_polynomial(irreps, tensor, 3, L)


def fixed_axis_angle_rotation(irreps: Irreps, axis: np.ndarray, angle: float) -> EquivariantPolynomial:
    """``input[u] -> output[u]``: rotation by a known angle about a known axis (reference ``rotations.py:23-46``)."""
    axis = np.asarray(axis, dtype=np.float64)
    axis = axis / np.linalg.norm(axis)

    def tensor(ir):
        D = _expm(float(angle) * np.einsum("a,aij->ij", axis, _rotation_generators(ir)))
        return _clean(D.T)  # (j, k)

    return _rotation_polynomial(irreps, tensor, 0, 0)


def inversion(irreps: Irreps) -> EquivariantPolynomial:
    """``input[u] -> output[u]``: the inversion ``x -> -x`` of O(3): every irrep times its parity (reference ``rotations.py:235-252``)."""
    if irreps.irrep_class.__name__ not in ("O3", "O3_e3nn"):
        raise ValueError(f"Unsupported irrep class {irreps.irrep_class.__name__}. Must be O3.")
    return _rotation_polynomial(irreps, lambda ir: float(ir.p) * np.eye(ir.dim), 0, 0)
