"""Identity of the reduced symmetric basis (not only its span) for the irreps of the benchmarked symmetric contraction.

``cue/reduced_basis.py`` restates the reference's algorithm
(``cuequivariance/group_theory/irreps_array/reduced_tensor_product.py:240-385,467-631,680-789``).  A basis of the
symmetric power is not unique, and learned weights refer to the reference's choice, so the span alone (equivariance,
rank, path counts) does not pin it.  What the reference's construction *defines*, read as mathematics, is rebuilt
here from nothing but the Clebsch-Gordan tensors (pinned against sympy in ``test_group_theory.py``) and numpy:

* power of one irrep: couple the factors with Clebsch-Gordan tensors (degree 3: first the symmetric square, then the
  third factor), keep the coefficient vectors for which the coupled tensor is symmetric under all permutations of its
  axes, and take Gram-Schmidt of the rows of the orthogonal projector onto that coefficient space in row order -
  what ``basis_intersection`` (``etc/linalg.py:182-235``) computes: ``gram_schmidt(x1 @ x1.T)`` of the null vectors of
  its block matrix is that projector times 1/2, whatever basis ``eigh`` returns.  For a one-dimensional space this fixes
  the sign: the first coefficient above 1e-5 is positive;
* sum of irreps: for every composition of the degree over the irreps (in the order of
  ``generate_tuples_with_fixed_sum``) couple the powers left to right, filter the output irreps at the last coupling,
  sum the distinct placements of the factors over the axes and divide by the square root of their number; concatenate
  and sort the output irreps stably.

The result is compared entry by entry (sign and normalisation included) with the restatement *before* its last step,
the greedy sparsifier (``etc/linalg.py:371-433``), for degrees 1 to 3 of ``0e+1o+2e+3o -> 0e+1o``, and for the
reference's documented ``lmax = 2`` case.  The sparsifier is a sequence of pairwise row replacements without a
definition apart from its own steps: the second test states which basis vectors it leaves untouched (pinned by the
above: all of degrees 1 and 2, 18 of the 20 of degree 3) and checks that each of the two it replaces is one pairwise
step from the canonical rows (the sparsest combination of two neighbouring rows).
"""

import itertools

import numpy as np
import pytest

from cuequivariance_amd import cue
from cuequivariance_amd.cue import reduced_basis as rb


def cg(a, b, c):
    w = cue.O3.clebsch_gordan(a, b, c)
    assert w.shape[0] == 1
    return w[0]


def regroup(entries):
    """entries: [(irrep, tensor)] in creation order -> [(irrep, [tensors])] sorted by irrep, creation order kept inside."""
    irs = sorted({ir for ir, _ in entries})
    return [(ir, [t for i, t in entries if i == ir]) for ir in irs]


def couple(b1, b2, keep):
    """Clebsch-Gordan coupling of two bases, in the segment order of reduce_basis_product (reduced_tensor_product.py:712-733)."""
    out = []
    for ir1, xs1 in b1:
        for ir2, xs2 in b2:
            for ir in ir1 * ir2:
                if keep is not None and ir not in keep:
                    continue
                c = cg(ir1, ir2, ir)
                for x1 in xs1:
                    for x2 in xs2:
                        out.append((ir, np.einsum("...i,...j,ijk->...k", x1, x2, c)))
    return regroup(out)


def symmetrise(t, n):
    return sum(np.transpose(t, p) for p in itertools.permutations(range(n))) / np.prod(range(1, n + 1))


def constrain_symmetric(basis, n, eps=1e-5):
    """Per output irrep: Gram-Schmidt (row order, threshold eps) of the projector onto the coefficient vectors whose
    combination of the coupled tensors is symmetric in its n axes."""
    out = []
    for ir, ts in basis:
        r = np.stack([t[..., 0].reshape(-1) for t in ts])  # component 0 decides, as in the reference
        np.testing.assert_allclose(r @ r.T, np.eye(len(ts)), atol=1e-12)  # orthonormal: x1 x1^T is then half the projector
        a = np.stack([(t[..., 0] - symmetrise(t[..., 0], n)).reshape(-1) for t in ts])
        w, v = np.linalg.eigh(a @ a.T)
        null = v[:, w < 1e-10]
        proj = null @ null.T
        q = []
        for i in range(proj.shape[0]):
            x = proj[i].copy()
            for u in q:
                x -= (u @ x) * u
            if np.linalg.norm(x) > eps:
                q.append(x / np.linalg.norm(x))
        for coeff in q:
            out.append((ir, sum(c * t for c, t in zip(coeff, ts))))
    return regroup(out)


def rule_product(keep, irs):
    return None if keep is None else frozenset(c for a in keep for b in irs for c in a * b)


def rule_power(irs, n):
    out = frozenset([cue.O3.trivial()])
    for _ in range(n):
        out = rule_product(out, irs)
    return out


def power_of_one_irrep(ir, n, keep):
    d = ir.dim
    eye = np.eye(d)
    if n == 1:
        return [(ir, [eye])] if keep is None or ir in keep else []
    x = [np.reshape(eye, (1,) * i + (d,) + (1,) * (n - i - 1) + (d,)) for i in range(n)]
    if n == 2:
        return constrain_symmetric(couple([(ir, [x[0]])], [(ir, [x[1]])], keep), 2)
    assert n == 3
    # the greedy merge takes axes (0, 1) first: every pair spans a symmetrised space of the same size and the first wins
    pair = power_of_one_irrep(ir, 2, rule_product(keep, [ir]))
    pair = [(i, [t.reshape(d, d, 1, -1) for t in ts]) for i, ts in pair]
    return constrain_symmetric(couple(pair, [(ir, [x[2]])], keep), 3)


def compositions(length, total):
    if length == 1:
        yield (total,)
        return
    for first in range(total, -1, -1):
        for rest in compositions(length - 1, total - first):
            yield (first,) + rest


def independent_basis(irs, degree, keep):
    """[(irrep, [tensors of shape (D,) * degree + (irrep.dim,)])] for the sum of the irreps ``irs`` (multiplicity one each)."""
    dims = [ir.dim for ir in irs]
    start = np.concatenate([[0], np.cumsum(dims)])
    D = int(start[-1])
    if degree == 1:
        out = []
        for i, ir in enumerate(irs):
            if ir in keep:
                t = np.zeros((D, ir.dim))
                t[start[i]: start[i + 1]] = np.eye(ir.dim)
                out.append((ir, t))
        return regroup(out)
    collected = []
    for term in compositions(len(irs), degree):
        which = [i for i, n in enumerate(term) if n]
        pw = [n for n in term if n]
        owner = tuple(i for i, n in zip(which, pw) for _ in range(n))
        factors, before = [], 0
        for i, n in zip(which, pw):
            f = power_of_one_irrep(irs[i], n, rule_product(keep, rule_power(irs, degree - n)))
            after = degree - before - n
            factors.append([(ir, [t.reshape((1,) * before + t.shape[:-1] + (1,) * after + t.shape[-1:]) for t in ts]) for ir, ts in f])
            before += n
        if len(factors) == 1:
            product = [(ir, ts) for ir, ts in factors[0] if ir in keep]
        else:
            cur = factors[0]
            for nxt in factors[1:-1]:
                cur = couple(cur, nxt, None)
            product = couple(cur, factors[-1], keep)
        for ir, ts in product:
            for t in ts:
                total, seen = np.zeros((D,) * degree + (ir.dim,)), set()
                for axes in itertools.permutations(range(degree)):
                    owners = tuple(owner[a] for a in axes)
                    if owners in seen:
                        continue
                    seen.add(owners)
                    window = tuple(slice(start[o], start[o + 1]) for o in owners)
                    total[window] += np.transpose(t, axes + (degree,))
                collected.append((ir, total / np.sqrt(len(seen))))
    return regroup(collected)


def columns(arr: rb.IrrepsArray):
    """[(irrep, [tensors])] of an IrrepsArray in mul_ir layout."""
    out = []
    for (mul, ir), seg in zip(arr.irreps, arr.segments):  # seg (..., mul, dim)
        out.append((ir, [seg[..., u, :] for u in range(mul)]))
    return out


CASES = [("0e+1o+2e+3o", "0e+1o", 3), ("0e+1o+2e", "0e+1o", 3)]


@pytest.mark.parametrize("irreps_in,irreps_out,max_degree", CASES)
def test_basis_before_sparsification_is_the_canonical_one(irreps_in, irreps_out, max_degree):
    irreps = cue.Irreps("O3", irreps_in)
    irs = [ir for _, ir in irreps]
    keep = frozenset(ir for _, ir in cue.Irreps("O3", irreps_out))
    for degree in range(1, max_degree + 1):
        got = rb._reduce_recursive((irreps,) * degree, rb._symmetric_perm_repr(degree), keep, 1e-5, True)
        want = independent_basis(irs, degree, keep)
        got_cols = columns(got)
        assert [(ir, len(ts)) for ir, ts in got_cols] == [(ir, len(ts)) for ir, ts in want], degree
        for (ir, a), (_, b) in zip(got_cols, want):
            for u, (x, y) in enumerate(zip(a, b)):
                # same vector, same sign, same normalisation (the restatement rounds to square roots of rationals: 1e-9)
                assert np.abs(x - y).max() <= 1e-9, (degree, ir, u, np.abs(x - y).max(), np.abs(x + y).max())
                # orthonormal per component: sum over the input axes of the squares is 1 for each output component
                np.testing.assert_allclose((y ** 2).sum(axis=tuple(range(degree))), 1.0, atol=1e-12)


def sparsest_combination(x0, x1):
    """The combination x0 - r x1 with the fewest non-zeros (brute force over the ratios that cancel an entry), or None
    when the two rows share no entry."""
    both = np.where((np.abs(x0) > 1e-12) & (np.abs(x1) > 1e-12))[0]
    best = None
    for r in sorted(set(np.round(x0[both] / x1[both], 9))):
        nnz = int((np.abs(x0 - r * x1) > 1e-9).sum())
        if best is None or nnz < best[0]:
            best = (nnz, r)
    return best


def test_what_the_sparsifier_changes_for_the_benchmarked_irreps():
    """Degrees 1 and 2: the published basis *is* the canonical one (the sparsifier finds nothing to do).  Degree 3: 18 of
    the 20 vectors (8 x 0e, 12 x 1o) are the canonical ones; the other two (1o, positions 6 and 10) are each ONE pairwise
    step of the sparsifier (``etc/linalg.py:325-368``) from the canonical rows: the combination of that row and its
    predecessor with the fewest non-zeros, scaled to the norm of the replaced row, positive coefficient on the first."""
    irreps = cue.Irreps("O3", "0e+1o+2e+3o")
    keep = frozenset(ir for _, ir in cue.Irreps("O3", "0e+1o"))
    touched = {}
    for degree in (1, 2, 3):
        pre = rb._reduce_recursive((irreps,) * degree, rb._symmetric_perm_repr(degree), keep, 1e-5, True)
        fin = rb.reduced_symmetric_tensor_product_basis(irreps, degree, keep_ir=keep)
        assert fin.irreps == pre.irreps
        for (ir, a), (_, b) in zip(columns(pre), columns(fin)):
            a2 = np.stack([t.reshape(-1) for t in a])
            b2 = np.stack([t.reshape(-1) for t in b])
            # published rows = q @ canonical rows (the canonical rows are orthonormal per component: q = b2 a2^T / dim)
            q = b2 @ a2.T / ir.dim
            np.testing.assert_allclose(q @ a2, b2, atol=1e-9)
            assert abs(np.linalg.det(q)) > 1e-6
            rows = [u for u in range(len(a)) if np.abs(b2[u] - a2[u]).max() > 1e-9]
            touched[(degree, str(ir))] = rows
            for u in rows:
                support = np.where(np.abs(q[u]) > 1e-9)[0]
                assert list(support) == [u - 1, u], (degree, ir, u, q[u])  # one step: this row and its predecessor
                nnz, r = sparsest_combination(a2[u - 1], a2[u])
                comb = a2[u - 1] - r * a2[u]
                comb *= np.linalg.norm(a2[u]) / np.linalg.norm(comb)
                assert nnz < int((np.abs(a2[u]) > 1e-12).sum())  # sparser than the row it replaces
                assert np.abs(b2[u] - comb).max() <= 1e-9 and q[u, u - 1] > 0
    assert touched == {(1, "0e"): [], (1, "1o"): [], (2, "0e"): [], (2, "1o"): [], (3, "0e"): [], (3, "1o"): [6, 10]}
