"""Change of basis that reduces a (permutation-symmetric) tensor power of a representation into irreps.

``reduced_symmetric_tensor_product_basis(irreps, degree, keep_ir=..., layout=...)`` returns an
:class:`IrrepsArray` ``U`` of shape ``(d, ..., d, irreps_out.dim)`` (``degree`` leading axes of extent
``d = irreps.dim``): column block ``(mul, ir)`` of the last axis maps the symmetric part of
``x ⊗ ... ⊗ x`` onto ``mul`` copies of ``ir``.

Restates the algorithm of ``cuequivariance/group_theory/irreps_array/reduced_tensor_product.py`` of the
reference: front ends ``:147-187``, recursion ``:240-385``, symmetric fast path ``:467-631``,
product/constraint helpers ``:680-789``, permutation bases ``:792-877``, rounding/sparsifying
``:880-903``; array container ``group_theory/irreps_array/numpy_irreps_array.py:27-293``.  Bases are not
unique; to obtain the reference's one (its learned weights refer to it) the numerical steps -
Clebsch-Gordan contraction order, eigen-decomposition, Gram-Schmidt sweep order, rounding, greedy
sparsification - are the reference's, in its order.
"""

from __future__ import annotations

import functools
import itertools
from math import prod
from typing import FrozenSet, Optional, Sequence, Tuple

import numpy as np

from . import linalg
from .irreps import Irrep, Irreps, IrrepsLayout, into_list_of_irrep

PermRepr = FrozenSet[Tuple[int, Tuple[int, ...]]]


# ---------------------------------------------------------------------------------------------
# selection rules (group_theory/representations/irrep.py:240-272)
# ---------------------------------------------------------------------------------------------
def selection_rule_product(irs1, irs2):
    """Irreps reachable from products ``ir1 * ir2``; ``None`` (no restriction) is absorbing."""
    if irs1 is None or irs2 is None:
        return None
    irs1 = [irs1] if isinstance(irs1, Irrep) else list(irs1)
    irs2 = [irs2] if isinstance(irs2, Irrep) else list(irs2)
    out = set()
    for a, b in itertools.product(irs1, irs2):
        out = out.union(a * b)
    return frozenset(out)


def selection_rule_power(irrep_class, irs, n: int):
    irs = [irs] if isinstance(irs, Irrep) else list(irs)
    out = frozenset([irrep_class.trivial()])
    for _ in range(n):
        out = selection_rule_product(out, irs)
    return out


# ---------------------------------------------------------------------------------------------
# array with an irreps-structured last axis (numpy_irreps_array.py:27-293)
# ---------------------------------------------------------------------------------------------
class IrrepsArray:
    """``array[..., irreps.dim]`` whose last axis is a concatenation of ``(mul, ir)`` blocks."""

    __slots__ = ("irreps", "array", "layout")

    def __init__(self, irreps: Irreps, array: np.ndarray, layout: IrrepsLayout = IrrepsLayout.mul_ir):
        if array.shape[-1] != irreps.dim:
            raise ValueError(f"Last dimension of array should be {irreps.dim}, got {array.shape[-1]}")
        self.irreps, self.array, self.layout = irreps, array, IrrepsLayout.as_layout(layout)

    @property
    def shape(self):
        return self.array.shape

    @property
    def segments(self) -> list:
        lead = self.array.shape[:-1]
        return [
            np.reshape(self.array[..., sl], lead + self.layout.shape(mi))
            for sl, mi in zip(self.irreps.slices(), self.irreps)
        ]

    @staticmethod
    def from_segments(irreps: Irreps, segments: Sequence[np.ndarray], layout, leading_shape) -> "IrrepsArray":
        layout = IrrepsLayout.as_layout(layout)
        if len(segments) != len(irreps):
            raise ValueError(f"Expected {len(irreps)} segments, got {len(segments)}")
        for seg, mi in zip(segments, irreps):
            if seg.shape[:-2] != tuple(leading_shape) or seg.shape[-2:] != layout.shape(mi):
                raise ValueError(f"segment of shape {seg.shape} does not fit {leading_shape} + {layout.shape(mi)}")
        if len(segments) > 0:
            array = np.concatenate(
                [np.reshape(seg, seg.shape[:-2] + (mi.mul * mi.ir.dim,)) for seg, mi in zip(segments, irreps)], axis=-1
            )
        else:
            array = np.empty(tuple(leading_shape) + (0,))
        return IrrepsArray(irreps, array, layout)

    @staticmethod
    def concatenate(arrays: Sequence["IrrepsArray"]) -> "IrrepsArray":
        if len(arrays) == 0:
            raise ValueError("Expected at least one input")
        cls = arrays[0].irreps.irrep_class
        irreps = Irreps(cls, [mi for a in arrays for mi in a.irreps])
        return IrrepsArray(irreps, np.concatenate([a.array for a in arrays], axis=-1), arrays[0].layout)

    def reshape(self, shape) -> "IrrepsArray":
        if shape[-1] not in (-1, self.irreps.dim):
            raise ValueError(f"Last dimension of shape should be -1 or {self.irreps.dim}, got {shape[-1]}")
        return IrrepsArray(self.irreps, self.array.reshape(shape), self.layout)

    def change_layout(self, layout) -> "IrrepsArray":
        layout = IrrepsLayout.as_layout(layout)
        if layout == self.layout:
            return self
        return IrrepsArray.from_segments(
            self.irreps, [np.moveaxis(s, -1, -2) for s in self.segments], layout, self.shape[:-1]
        )

    def sort(self) -> "IrrepsArray":
        s = self.irreps.sort()
        segs = self.segments
        return IrrepsArray.from_segments(s.irreps, [segs[i] for i in s.inv], self.layout, self.shape[:-1])

    def simplify(self) -> "IrrepsArray":
        if self.layout == IrrepsLayout.mul_ir:
            return IrrepsArray(self.irreps.simplify(), self.array, self.layout)
        return self.change_layout(IrrepsLayout.mul_ir).simplify().change_layout(self.layout)

    def regroup(self) -> "IrrepsArray":
        return self.sort().simplify()

    def filter(self, *, keep) -> "IrrepsArray":
        if keep is None:
            return self
        keep = into_list_of_irrep(self.irreps.irrep_class, keep)
        return IrrepsArray.from_segments(
            self.irreps.filter(keep=keep),
            [seg for seg, mi in zip(self.segments, self.irreps) if mi.ir in keep],
            self.layout,
            self.shape[:-1],
        )

    def __repr__(self):
        return f"IrrepsArray({self.irreps}, shape={self.shape}, {self.layout})"


# ---------------------------------------------------------------------------------------------
# front ends (reduced_tensor_product.py:56-237)
# ---------------------------------------------------------------------------------------------
def _symmetric_perm_repr(n: int) -> PermRepr:
    return frozenset((1, p) for p in itertools.permutations(range(n)))


def _antisymmetric_perm_repr(n: int) -> PermRepr:
    return frozenset((linalg.perm_sign(p), p) for p in itertools.permutations(range(n)))


def _keep_set(irreps: Irreps, keep_ir):
    if keep_ir is None:
        return None
    return frozenset(into_list_of_irrep(irreps.irrep_class, keep_ir))


def reduced_symmetric_tensor_product_basis(irreps: Irreps, degree: int, *, layout=IrrepsLayout.mul_ir,
                                           epsilon: float = 1e-5, keep_ir=None,
                                           _use_optimized_implementation: bool = True) -> IrrepsArray:
    """Basis of the fully symmetric part of ``irreps ** degree`` (reduced_tensor_product.py:147-187)."""
    assert isinstance(irreps, Irreps)
    return _entrypoint((irreps,) * degree, _symmetric_perm_repr(degree), _keep_set(irreps, keep_ir),
                       IrrepsLayout.as_layout(layout), epsilon, _use_optimized_implementation)


def reduced_antisymmetric_tensor_product_basis(irreps: Irreps, degree: int, *, layout=IrrepsLayout.mul_ir,
                                               epsilon: float = 1e-5, keep_ir=None,
                                               _use_optimized_implementation: bool = True) -> IrrepsArray:
    """Basis of the fully antisymmetric part of ``irreps ** degree`` (reduced_tensor_product.py:194-237)."""
    assert isinstance(irreps, Irreps)
    return _entrypoint((irreps,) * degree, _antisymmetric_perm_repr(degree), _keep_set(irreps, keep_ir),
                       IrrepsLayout.as_layout(layout), epsilon, _use_optimized_implementation)


def reduced_tensor_product_basis(formula_or_irreps_list, *, layout=IrrepsLayout.mul_ir, epsilon: float = 1e-5,
                                 keep_ir=None, _use_optimized_implementation: bool = True, **irreps_dict) -> IrrepsArray:
    """Basis of a tensor product under the index symmetries of a formula such as ``"ijk=jik=ikj"`` or
    ``"ij=-ji"``, or of a plain list of irreps without symmetry (reduced_tensor_product.py:56-141)."""
    layout = IrrepsLayout.as_layout(layout)
    if isinstance(formula_or_irreps_list, (tuple, list)):
        irreps_tuple = tuple(formula_or_irreps_list)
        assert all(isinstance(x, Irreps) for x in irreps_tuple)
        perm_repr = frozenset({(1, tuple(range(len(irreps_tuple))))})
        return _entrypoint(irreps_tuple, perm_repr, _keep_set(irreps_tuple[0], keep_ir), layout, epsilon,
                           _use_optimized_implementation)

    f0, perm_repr = germinate_perm_repr(formula_or_irreps_list)
    assert all(isinstance(x, Irreps) for x in irreps_dict.values())
    for name in irreps_dict:
        if len(name) != 1:
            raise TypeError(f"got an unexpected keyword argument '{name}'")
    # indices exchanged by a permutation carry the same irreps
    for _sign, p in perm_repr:
        f = "".join(f0[i] for i in p)
        for a, b in zip(f0, f):
            if a in irreps_dict and b in irreps_dict and irreps_dict[a] != irreps_dict[b]:
                raise RuntimeError(f"irreps of {a} and {b} should be the same")
            if a in irreps_dict:
                irreps_dict[b] = irreps_dict[a]
            if b in irreps_dict:
                irreps_dict[a] = irreps_dict[b]
    for a in f0:
        if a not in irreps_dict:
            raise RuntimeError(f"index {a} has no irreps associated to it")
    for a in irreps_dict:
        if a not in f0:
            raise RuntimeError(f"index {a} has an irreps but does not appear in the fomula")
    irreps_tuple = tuple(irreps_dict[a] for a in f0)
    return _entrypoint(irreps_tuple, perm_repr, _keep_set(irreps_tuple[0], keep_ir), layout, epsilon,
                       _use_optimized_implementation)


@functools.lru_cache(maxsize=None)
def germinate_perm_repr(formula: str):
    """Close the signed permutations named by a formula under inversion and composition
    (reduced_tensor_product.py:637-677)."""
    parts = [(-1 if f.startswith("-") else 1, f.replace("-", "")) for f in formula.split("=")]
    s0, f0 = parts[0]
    assert s0 == 1
    for _s, f in parts:
        if len(set(f)) != len(f) or set(f) != set(f0):
            raise RuntimeError(f"{f} is not a permutation of {f0}")
        if len(f0) != len(f):
            raise RuntimeError(f"{f0} and {f} don't have the same number of indices")
    group = {(s, tuple(f.index(i) for i in f0)) for s, f in parts}
    while True:
        n = len(group)
        group = group.union([(s, linalg.perm_inverse(p)) for s, p in group])
        group = group.union([(s1 * s2, linalg.perm_compose(p1, p2)) for s1, p1 in group for s2, p2 in group])
        if len(group) == n:
            break
    return f0, frozenset(group)


# ---------------------------------------------------------------------------------------------
# back end (reduced_tensor_product.py:243-385)
# ---------------------------------------------------------------------------------------------
def _entrypoint(irreps_tuple, perm_repr, keep_ir, layout, epsilon, optimized) -> IrrepsArray:
    out = _reduce_recursive(irreps_tuple, perm_repr, keep_ir, epsilon, optimized)
    out = _sparsify(out)  # sparsifying only once, at the end, sparsifies best
    if layout == IrrepsLayout.ir_mul:
        x = out.array
        for axis, irreps in enumerate(irreps_tuple + (out.irreps,)):
            x = np.moveaxis(x, axis, -1)
            x = IrrepsArray(irreps, x, IrrepsLayout.mul_ir).change_layout(IrrepsLayout.ir_mul).array
            x = np.moveaxis(x, -1, axis)
        return IrrepsArray(out.irreps, x, IrrepsLayout.ir_mul)
    return out


@functools.lru_cache(maxsize=None)
def _reduce_recursive(irreps_tuple, perm_repr: PermRepr, keep_ir, epsilon: float, optimized: bool) -> IrrepsArray:
    degree = len(irreps_tuple)
    if optimized and degree > 1 and perm_repr == _symmetric_perm_repr(degree) and irreps_tuple[0].num_irreps > 1:
        return _rounded(_symmetric_power_by_terms(irreps_tuple[0], degree, epsilon=epsilon, keep_ir=keep_ir))

    dims = tuple(irreps.dim for irreps in irreps_tuple)
    # one identity basis per index, broadcastable against the others
    bases = [
        (
            frozenset({i}),
            IrrepsArray(irreps, np.reshape(np.eye(irreps.dim), (1,) * i + (irreps.dim,) + (1,) * (degree - i - 1) + (irreps.dim,))),
        )
        for i, irreps in enumerate(irreps_tuple)
    ]
    while True:
        if len(bases) == 0:
            raise RuntimeError("Tensor Product raised to the 0th power is not defined.")
        if len(bases) == 1:
            f, b = bases[0]
            assert f == frozenset(range(degree))
            if keep_ir is not None:
                b = b.filter(keep=keep_ir)
            return b.regroup()
        if len(bases) == 2:
            (fa, a), (fb, b) = bases
            f = frozenset(fa | fb)
            ab = reduce_basis_product(a, b, keep_ir)
            if len(subrepr_permutation(f, perm_repr)) == 1:
                return ab.regroup()
            p = reduce_subgroup_permutation(f, perm_repr, dims)
            ab = constrain_rotation_basis_by_permutation_basis(ab, p, epsilon=epsilon)
            return _rounded(ab.regroup())

        # greedy: merge the pair of index sets whose symmetrised space is smallest
        smallest, best = np.inf, None
        for i in range(len(bases)):
            for j in range(i + 1, len(bases)):
                f = frozenset(bases[i][0] | bases[j][0])
                p_dim = reduce_subgroup_permutation(f, perm_repr, dims, return_dim=True)
                if p_dim < smallest:
                    smallest, best = p_dim, (i, j, f)
        i, j, f = best
        del bases[j]
        del bases[i]
        sub_irreps = tuple(irreps_tuple[k] for k in f)
        sub_perm_repr = subrepr_permutation(f, perm_repr)
        keep = keep_ir
        for k, irreps in enumerate(irreps_tuple):
            if k not in f:
                keep = selection_rule_product(keep, {ir for _, ir in irreps})
        ab = _reduce_recursive(sub_irreps, sub_perm_repr, keep, epsilon, optimized)
        ab = ab.reshape(tuple(dims[k] if k in f else 1 for k in range(degree)) + (-1,))
        bases = [(f, ab)] + bases


# ---------------------------------------------------------------------------------------------
# symmetric power of a sum of irreps, term by term (reduced_tensor_product.py:391-631)
# ---------------------------------------------------------------------------------------------
def _compositions(length: int, total: int):
    """Non-negative integer tuples of the given length and sum, first entry descending."""
    if length == 1:
        yield (total,)
        return
    if total == 0:
        yield (0,) * length
        return
    for first in range(total, -1, -1):
        for rest in _compositions(length - 1, total - first):
            yield (first,) + rest


def _offsets_before(seq):
    return np.cumsum([0, *seq])[:-1]


def _offsets_after(seq):
    return _offsets_before(seq[::-1])[::-1]


def _symmetric_power_by_terms(irreps: Irreps, degree: int, *, epsilon: float, keep_ir) -> IrrepsArray:
    """``(ir_1 + ... + ir_m) ** degree`` restricted to symmetric tensors: for every way of choosing powers
    ``(n_1, ..., n_m)`` summing to ``degree``, couple the symmetric powers ``ir_i ** n_i`` and average the result over
    the distinct placements of the factors among the ``degree`` axes."""
    cls = irreps.irrep_class
    irreps = Irreps(cls, [(1, ir) for mul, ir in irreps for _ in range(mul)])
    block_dims = [mul * ir.dim for mul, ir in irreps]
    before, after = _offsets_before(block_dims), _offsets_after(block_dims)

    powers = {}
    for i, mul_ir in enumerate(irreps):
        powers[i] = [IrrepsArray(Irreps(cls, [cls.trivial()]), np.asarray([1.0]))]
        for n in range(1, degree + 1):
            powers[i].append(
                reduced_symmetric_tensor_product_basis(
                    Irreps(cls, [mul_ir]),
                    n,
                    epsilon=epsilon,
                    keep_ir=selection_rule_product(
                        keep_ir, selection_rule_power(cls, {ir for _, ir in irreps}, degree - n)
                    ),
                )
            )

    collected = []
    for term in _compositions(len(irreps), degree):
        which = [i for i, n in enumerate(term) if n != 0]
        pw = [n for n in term if n != 0]
        axis_owner = tuple(i for i, n in zip(which, pw) for _ in range(n))  # irrep index owning each axis

        # give every factor the full set of `degree` leading axes (extent 1 where it does not act)
        lead_before, lead_after = _offsets_before(pw), _offsets_after(pw)
        factors = []
        for pos, (i, n) in enumerate(zip(which, pw)):
            t = powers[i][n]
            factors.append(t.reshape((1,) * lead_before[pos] + t.shape[:-1] + (1,) * lead_after[pos] + t.shape[-1:]))

        if len(factors) == 1:
            product = factors[0].filter(keep=keep_ir)
        else:
            cur = factors[0]
            for nxt in factors[1:-1]:
                cur = reduce_basis_product(cur, nxt)
            product = reduce_basis_product(cur, factors[-1], keep_ir=keep_ir)
        if product.irreps.dim == 0:
            continue

        shape = (irreps.dim,) * degree + (product.irreps.dim,)
        total = np.zeros_like(product.array, shape=shape)
        seen = set()
        for axes in itertools.permutations(range(len(axis_owner))):
            owners = tuple(axis_owner[a] for a in axes)
            if owners in seen:
                continue
            seen.add(owners)
            moved = np.transpose(product.array, axes + (len(axes),))
            window = tuple(slice(before[o], irreps.dim - after[o]) for o in owners) + (slice(0, shape[-1]),)
            total[window] += moved
        collected.append(IrrepsArray(product.irreps, total / np.sqrt(len(seen))))

    return IrrepsArray.concatenate(collected).regroup()


# ---------------------------------------------------------------------------------------------
# coupling two bases, imposing the permutation symmetry (reduced_tensor_product.py:680-877)
# ---------------------------------------------------------------------------------------------
_product_cache: dict = {}


def reduce_basis_product(basis1: IrrepsArray, basis2: IrrepsArray, keep_ir=None) -> IrrepsArray:
    """Couple every block of ``basis1`` with every block of ``basis2`` through Clebsch-Gordan coefficients."""
    basis1, basis2 = basis1.regroup(), basis2.regroup()
    assert basis1.layout == basis2.layout
    layout = basis1.layout
    if keep_ir is not None:
        keep_ir = frozenset(keep_ir)
    assert basis1.array.dtype == np.float64 and basis2.array.dtype == np.float64
    key = (keep_ir, basis1.irreps, basis2.irreps, basis1.shape, basis2.shape,
           hash(basis1.array.tobytes()), hash(basis2.array.tobytes()))
    if key in _product_cache:
        return _product_cache[key]

    out_irreps, out_segments = [], []
    for (mul1, ir1), x1 in zip(basis1.irreps, basis1.segments):
        for (mul2, ir2), x2 in zip(basis2.irreps, basis2.segments):
            for ir in ir1 * ir2:
                if keep_ir is not None and ir not in keep_ir:
                    continue
                cg = ir1.clebsch_gordan(ir1, ir2, ir)
                if layout == IrrepsLayout.mul_ir:
                    x = np.einsum("...ui,...vj,wijk->...uvwk", x1, x2, cg)
                else:
                    x = np.einsum("...iu,...jv,wijk->...kuvw", x1, x2, cg)
                m = mul1 * mul2 * len(cg)
                out_segments.append(np.reshape(x, x.shape[:-4] + layout.shape((m, ir))))
                out_irreps.append((m, ir))
    irreps = Irreps(basis1.irreps.irrep_class, out_irreps)
    lead = np.broadcast_shapes(basis1.shape[:-1], basis2.shape[:-1])
    out = IrrepsArray.from_segments(irreps, out_segments, layout, lead).regroup()
    _product_cache[key] = out
    return out


def constrain_rotation_basis_by_permutation_basis(rotation_basis: IrrepsArray, permutation_basis: np.ndarray, *,
                                                  epsilon: float = 1e-5, round_fn=lambda x: x) -> IrrepsArray:
    """Keep, irrep by irrep, the part of a rotation basis that lies in the span of a permutation basis."""
    assert rotation_basis.shape[:-1] == permutation_basis.shape[1:]
    assert rotation_basis.layout == IrrepsLayout.mul_ir
    perm = np.reshape(permutation_basis, (permutation_basis.shape[0], prod(permutation_basis.shape[1:])))

    out_irreps, out_segments = [], []
    segs = rotation_basis.segments
    for ir in sorted({ir for _, ir in rotation_basis.irreps}):
        idx = [i for i, (_, ir_) in enumerate(rotation_basis.irreps) if ir == ir_]
        rot = np.concatenate([segs[i] for i in idx], axis=-2)
        mul = rot.shape[-2]
        R = np.reshape(rot[..., 0], (-1, mul)).T  # (mul, dim): first component identifies the copy
        # rows of perm do not share non-zero columns, so those not touching R's support cannot matter
        perm_used = perm[~np.all(perm[:, ~np.all(R == 0, axis=0)] == 0, axis=1)]
        P, _ = linalg.basis_intersection(R, perm_used, epsilon=epsilon, round_fn=round_fn)
        out_irreps.append((len(P), ir))
        out_segments.append(round_fn(np.einsum("vu,...ui->...vi", P, rot)))
    irreps = Irreps(rotation_basis.irreps.irrep_class, out_irreps)
    return IrrepsArray.from_segments(irreps, out_segments, IrrepsLayout.mul_ir, rotation_basis.shape[:-1])


def subrepr_permutation(sub: FrozenSet[int], perm_repr: PermRepr) -> PermRepr:
    """The permutations that move only indices of ``sub``, renumbered onto ``range(len(sub))``."""
    order = sorted(sub)
    return frozenset(
        {
            (s, tuple(order.index(i) for i in p if i in sub))
            for s, p in perm_repr
            if all(i in sub or i == j for j, i in enumerate(p))
        }
    )


def reduce_subgroup_permutation(sub: FrozenSet[int], perm_repr: PermRepr, dims, return_dim: bool = False):
    sub_perm = subrepr_permutation(sub, perm_repr)
    sub_dims = tuple(dims[i] for i in sub)
    if len(sub_perm) == 1:
        if return_dim:
            return prod(sub_dims)
        return np.eye(prod(sub_dims)).reshape((prod(sub_dims),) + sub_dims)
    base = reduce_permutation_base(sub_perm, sub_dims)
    if return_dim:
        return len(base)
    basis = reduce_permutation_matrix(base, sub_dims)
    return np.reshape(basis, (-1,) + tuple(dims[i] if i in sub else 1 for i in range(len(dims))))


@functools.lru_cache(maxsize=None)
def _all_multi_indices(dims):
    return list(itertools.product(*(range(d) for d in dims)))


@functools.lru_cache(maxsize=None)
def reduce_permutation_base(perm_repr: PermRepr, dims):
    """Orbits of tensor entries under the signed permutations; an entry related to minus itself is dropped.
    Each orbit is stored with both overall signs (the sign is fixed later)."""
    base = set()
    for x in _all_multi_indices(dims):
        orbit = {(s, tuple(x[i] for i in p)) for s, p in perm_repr}
        if (-1, x) not in orbit:
            base.add(frozenset({frozenset(orbit), frozenset({(-s, y) for s, y in orbit})}))
    return frozenset(base)


@functools.lru_cache(maxsize=None)
def reduce_permutation_matrix(base, dims) -> np.ndarray:
    """Orthonormal rows, one per orbit, in the flattened full tensor space."""
    base = sorted([sorted([sorted(xs) for xs in x]) for x in base])
    Q = np.zeros((len(base), prod(dims)), np.float64)
    for row, x in enumerate(base):
        x = max(x, key=lambda xs: sum(s for s, _ in xs))
        for s, e in x:
            col = 0
            for k, d in zip(e, dims):
                col = col * d + k
            Q[row, col] = s / len(x) ** 0.5
    np.testing.assert_allclose(Q @ Q.T, np.eye(len(base)))
    return Q.reshape(len(base), *dims)


def _rounded(x: IrrepsArray) -> IrrepsArray:
    return IrrepsArray(x.irreps, linalg.round_to_sqrt_rational(x.array), x.layout)


def _sparsify(x: IrrepsArray) -> IrrepsArray:
    assert x.layout == IrrepsLayout.mul_ir
    x = x.regroup()
    segments = []
    for seg in x.segments:
        seg = np.moveaxis(seg, -2, 0)  # (mul, ...)
        seg, _, _ = linalg.sparsify_matrix(seg, round_fn=linalg.round_to_sqrt_rational)
        segments.append(np.moveaxis(seg, 0, -2))
    return IrrepsArray.from_segments(x.irreps, segments, IrrepsLayout.mul_ir, x.shape[:-1])
