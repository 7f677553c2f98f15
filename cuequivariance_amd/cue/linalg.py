"""Numerical helpers of the reduced tensor-product basis: rounding to ``sqrt(n/d)``, Gram-Schmidt,
intersection of two row spaces, row sparsification, permutation utilities.

Restates ``cuequivariance/etc/linalg.py:30-433`` of the reference.  The floating-point operations are
kept in the reference's order on purpose: the basis they produce feeds learned weights, so the same
input must give the same numbers, not merely an equivalent basis.
"""

from __future__ import annotations

import itertools

import networkx
import numpy as np

MAX_DENOMINATOR = 2**40  # leaves room below the 53-bit mantissa for numerical noise


# ---------------------------------------------------------------------------------------------
# rounding (etc/linalg.py:30-168)
# ---------------------------------------------------------------------------------------------
def _reduce_fraction(n, d):
    g = np.gcd(n, d)
    g = np.where(d < 0, -g, g)
    return n // g, d // g


def _ratio_in_unit_interval(x):
    """(n, d) with n/d ~ x for 0 < x <= 1; (0, 0) when x underflows."""
    big = 1 << 62
    n = np.floor(x * big).astype(np.int64)
    d = np.round(n / x).astype(np.int64)
    return n, d


def approx_integer_ratio(x):
    """Element-wise integer ratio of a float64 array; ``d == 0`` marks values too small or too large."""
    x = np.asarray(x, dtype=np.float64)
    sign = np.sign(x).astype(np.int64)
    x = np.abs(x)
    n, d = np.zeros_like(x, np.int64), np.ones_like(x, np.int64)
    small = (x > 0.0) & (x <= 1.0)
    n, d = np.where(small, _ratio_in_unit_interval(np.where(small, x, 1.0)), (n, d))
    large = x > 1.0
    n, d = np.where(large, _ratio_in_unit_interval(1 / np.where(large, x, 1.0))[::-1], (n, d))
    ok = d > 0
    n, d = np.where(ok, _reduce_fraction(sign * n, np.where(ok, d, 1)), (n, d))
    return n, d


def limit_denominator(n, d, max_denominator: int):
    """Vectorised ``fractions.Fraction.limit_denominator`` on reduced fractions with ``d > 0``."""
    n = np.asarray(n, dtype=np.int64)
    d = np.asarray(d, dtype=np.int64)
    n0, d0 = n, d
    p0, q0, p1, q1 = np.zeros_like(n), np.ones_like(n), np.ones_like(n), np.zeros_like(n)
    while True:
        a = n // d
        q2 = q0 + a * q1
        stop = (q2 > max_denominator) | (d0 <= max_denominator)
        if np.all(stop):
            break
        p0, q0, p1, q1 = np.where(stop, (p0, q0, p1, q1), (p1, q1, p0 + a * p1, q2))
        n, d = np.where(stop, (n, d), (d, n - a * d))
    with np.errstate(divide="ignore"):
        k = (max_denominator - q0) // q1
    n1, d1 = p0 + k * p1, q0 + k * q1
    n2, d2 = p1, q1
    with np.errstate(over="ignore"):
        # the products wrap around int64, their differences do not (bounded by d0)
        closer2 = np.abs(d1 * (n2 * d0 - n0 * d2)) <= np.abs(d2 * (n1 * d0 - n0 * d1))
    return np.where(d0 <= max_denominator, (n0, d0), np.where(closer2, (n2, d2), (n1, d1)))


def _real_and_imag(f):
    def wrapped(x, *a, **k):
        if np.iscomplex(x).any():
            return f(np.real(x), *a, **k) + 1j * f(np.imag(x), *a, **k)
        return f(x, *a, **k)

    return wrapped


@_real_and_imag
def round_to_sqrt_rational(x, max_denominator: int = MAX_DENOMINATOR):
    """Closest number of the form ``±sqrt(n/d)`` with ``d <= max_denominator``."""
    x = np.asarray(x, dtype=np.float64)
    sign = np.sign(x)
    n, d = approx_integer_ratio(x**2)
    ok = d > 0
    n, d = limit_denominator(n, np.where(ok, d, 1), max_denominator)
    return np.where(ok, sign * np.sqrt(n / d), 0.0)


# ---------------------------------------------------------------------------------------------
# subspaces (etc/linalg.py:171-246)
# ---------------------------------------------------------------------------------------------
def _identity(x):
    return x


def gram_schmidt(A: np.ndarray, *, epsilon: float = 1e-5, round_fn=_identity) -> np.ndarray:
    """Orthonormal rows spanning the rows of ``A`` (rows of norm below ``epsilon`` after projection are dropped).

    Works in place on the rows of ``A`` like the reference does.
    """
    assert A.ndim == 2 and A.dtype in (np.float64, np.complex128)
    kept = []
    for r in range(A.shape[0]):
        v = A[r]
        for q in kept:
            v -= np.dot(np.conj(q), v) * q
        nrm = np.linalg.norm(v)
        if nrm > epsilon:
            kept.append(round_fn(v / nrm))
    return np.stack(kept) if kept else np.empty((0, A.shape[1]))


def basis_intersection(basis1: np.ndarray, basis2: np.ndarray, *, epsilon: float = 1e-5, round_fn=_identity):
    """Projectors ``(P1, P2)`` such that ``P1 @ basis1`` (= ``P2 @ basis2`` up to basis choice) spans the
    intersection of the two row spaces: null space of the Gram matrix of ``[basis1; -basis2]``."""
    assert basis1.ndim == 2 and basis2.ndim == 2 and basis1.shape[1] == basis2.shape[1]
    n1 = basis1.shape[0]
    gram = np.concatenate(
        [
            np.concatenate([basis1 @ basis1.T, -basis1 @ basis2.T], axis=1),
            np.concatenate([-basis2 @ basis1.T, basis2 @ basis2.T], axis=1),
        ],
        axis=0,
    )
    gram = round_fn(gram)
    w, v = np.linalg.eigh(gram)
    v = v[:, w < epsilon]
    x1 = v[:n1, :]
    x1 = gram_schmidt(x1 @ x1.T, epsilon=epsilon, round_fn=round_fn)
    x2 = v[n1:, :]
    x2 = gram_schmidt(x2 @ x2.T, epsilon=epsilon, round_fn=round_fn)
    return x1, x2


# ---------------------------------------------------------------------------------------------
# permutations (etc/linalg.py:249-292)
# ---------------------------------------------------------------------------------------------
def perm_compose(p1, p2):
    return tuple(p1[p2[i]] for i in range(len(p1)))


def perm_inverse(p):
    return tuple(p.index(i) for i in range(len(p)))


def perm_sign(p) -> int:
    seen, sign = set(), 1
    for start in range(len(p)):
        if start in seen:
            continue
        length, i = 0, start
        while i not in seen:
            seen.add(i)
            i = p[i]
            length += 1
        if length % 2 == 0:
            sign = -sign
    return sign


def triu_array(x: np.ndarray, ndim: int) -> np.ndarray:
    """Fold a tensor that is contracted with ``ndim`` identical operands onto sorted leading indices."""
    idx = np.nonzero(x)
    vals = x[idx]
    idx = np.stack(idx, axis=1)
    idx = np.concatenate([np.sort(idx[:, :ndim], axis=1), idx[:, ndim:]], axis=1)
    idx, inverse = np.unique(idx, axis=0, return_inverse=True)
    vals = np.bincount(inverse.reshape(-1), vals)
    out = np.zeros_like(x)
    out[tuple(idx.T)] = vals
    return out


# ---------------------------------------------------------------------------------------------
# sparsification (etc/linalg.py:295-433)
# ---------------------------------------------------------------------------------------------
def _sparser_combination(row0: np.ndarray, row1: np.ndarray, round_fn):
    """None if the rows share no column; ``("keep",)`` if no combination is sparser; else
    ``("replace", a0, a1, new_row, which)`` with ``new_row = a0*row0 + a1*row1`` replacing row ``which``."""
    both = np.where((row0 != 0) & (row1 != 0))[0]
    if len(both) == 0:
        return None
    ratios = round_fn(row0[both] / row1[both])
    ratios, counts = np.unique(ratios, return_counts=True)
    r, nc = ratios[np.argmax(counts)], np.max(counts)
    only0 = np.sum((row0 != 0) & (row1 == 0))
    only1 = np.sum((row0 == 0) & (row1 != 0))
    if nc > min(only0, only1):
        res = row0 - r * row1
        which = 1 if only0 < only1 else 0
        v = np.linalg.norm(row0 if which == 0 else row1) / np.linalg.norm(res)
        res = round_fn(res * v)
        return ("replace", v, -r * v, res, which)
    return ("keep",)


def sparsify_matrix(x_in: np.ndarray, max_iterations: int = 20, round_fn=_identity):
    """Greedy pairwise row combinations that lower the number of non-zeros.  Returns ``(q @ x, q, graph)``."""
    row_shape = x_in.shape[1:]
    flat = np.reshape(x_in, (len(x_in), int(np.prod(row_shape))))
    cols = np.where(np.any(flat != 0, axis=0))[0]
    x = flat[:, cols]
    q = np.eye(x.shape[0])

    graph = networkx.Graph()
    graph.add_nodes_from(range(x.shape[0]))
    for i0, i1 in itertools.combinations(range(x.shape[0]), 2):
        graph.add_edge(i0, i1)

    it, progress = 0, True
    while progress and it < max_iterations:
        progress = False
        nxt = networkx.Graph()
        nxt.add_nodes_from(range(x.shape[0]))
        for i0, i1 in graph.edges:
            res = _sparser_combination(x[i0], x[i1], round_fn)
            if res is None:
                continue
            if res[0] == "keep":
                nxt.add_edge(i0, i1)
                continue
            _, a0, a1, row, which = res
            progress = True
            target = i0 if which == 0 else i1
            x[target] = row
            q[target] = a0 * q[i0] + a1 * q[i1]
            nxt.add_edge(i0, i1)
            for i in graph.neighbors(i0):
                if i != i1:
                    nxt.add_edge(i, i1)
            for i in graph.neighbors(i1):
                if i != i0:
                    nxt.add_edge(i, i0)
        it += 1
        graph = nxt

    out = np.zeros_like(flat)
    out[:, cols] = x
    return np.reshape(out, (len(out),) + row_shape), q, graph
