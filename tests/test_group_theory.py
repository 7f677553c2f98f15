"""Pins the group-theory layer (irreps, Clebsch-Gordan, spherical harmonics) without the reference.

Checks are chosen so that a plausible mistake (a wrong sign or phase, a transposed operand, a
dropped normalisation) fails one of them:

* SU(2) coefficients against sympy's independent implementation (all j <= 3, half-integers too);
* the intertwiner identity with the Lie-algebra generators, as the reference tests it
  (``cuequivariance/tests/group_theory/clebsch_gordan_test.py:23-35``);
* textbook special cases (1 x 1 -> 0 is the dot product, 1 x 1 -> 1 the cross product);
* documented values of the reference (sort example ``irreps.py``, spherical harmonics at (0,1,0)
  from ``cuequivariance_jax/.../segmented_polynomial.py:112-117``, norm and equivariance as in
  ``cuequivariance/tests/group_theory/equivariant_polynomial_test.py:55-72``).
"""

import itertools

import numpy as np
import pytest

from cuequivariance_amd import cue


def test_su2_clebsch_gordan_matches_sympy():
    from sympy import Rational
    from sympy.physics.quantum.cg import CG

    twos = range(0, 7)  # 2j = 0..6
    checked = 0
    for tj1, tj2 in itertools.product(twos, twos):
        for tj3 in range(abs(tj1 - tj2), tj1 + tj2 + 1, 2):
            if tj3 > 6:
                continue
            c = cue.SU2.clebsch_gordan(cue.SU2(tj1 / 2), cue.SU2(tj2 / 2), cue.SU2(tj3 / 2))[0]
            for a in range(tj1 + 1):
                for b in range(tj2 + 1):
                    tm1, tm2 = -tj1 + 2 * a, -tj2 + 2 * b
                    tm3 = tm1 + tm2
                    if abs(tm3) > tj3:
                        continue
                    ref = CG(Rational(tj1, 2), Rational(tm1, 2), Rational(tj2, 2), Rational(tm2, 2),
                             Rational(tj3, 2), Rational(tm3, 2)).doit()
                    assert abs(float(ref) - c[a, b, (tj3 + tm3) // 2]) < 1e-12
                    checked += 1
    assert checked > 500


def test_su2_normalisation():
    # sum over (m1, m2) of C^2 is 1 for each m3: the tensor is NOT divided by sqrt(2 j3 + 1)
    for j1, j2 in [(1, 1), (2, 1), (3, 2), (1.5, 0.5)]:
        for ir3 in cue.SU2(j1) * cue.SU2(j2):
            c = cue.SU2.clebsch_gordan(cue.SU2(j1), cue.SU2(j2), ir3)[0]
            np.testing.assert_allclose((c**2).sum(axis=(0, 1)), np.ones(ir3.dim), atol=1e-12)


@pytest.mark.parametrize("Group", [cue.SU2, cue.SO3, cue.O3])
def test_clebsch_gordan_intertwiner(Group):
    it = Group.iterator()
    irreps = [next(it) for _ in range(6 if Group is cue.O3 else 4)]
    for r1, r2, r3 in itertools.combinations_with_replacement(irreps, 3):
        C = Group.clebsch_gordan(r1, r2, r3)
        a1 = np.einsum("zijk,giu->gzujk", C, r1.X)
        a2 = np.einsum("zijk,gju->gziuk", C, r2.X)
        a3 = np.einsum("zijk,guk->gziju", C, r3.X)
        np.testing.assert_allclose(a1 + a2, a3, atol=1e-10, rtol=0)


def test_so3_generators_are_real_antisymmetric_and_close():
    for ell in range(4):
        X = cue.SO3(ell).X
        np.testing.assert_allclose(X, -np.swapaxes(X, 1, 2), atol=1e-12)
        # [X0, X1] = +/- X2 up to the structure constants: the algebra closes
        comm = X[0] @ X[1] - X[1] @ X[0]
        coeffs = [np.vdot(X[k], comm) / max(np.vdot(X[k], X[k]), 1e-30) for k in range(3)]
        np.testing.assert_allclose(comm, sum(c * X[k] for k, c in enumerate(coeffs)), atol=1e-10)


def test_real_cg_special_cases():
    one = cue.O3(1, -1)
    dot = cue.O3.clebsch_gordan(one, one, cue.O3(0, 1))[0][:, :, 0]
    assert abs(abs(dot[0, 0]) - 1 / np.sqrt(3)) < 1e-12
    np.testing.assert_allclose(dot, dot[0, 0] * np.eye(3), atol=1e-12)
    cross = cue.O3.clebsch_gordan(one, one, cue.O3(1, 1))[0]
    eps = np.zeros((3, 3, 3))
    for i, j, k in itertools.permutations(range(3)):
        eps[i, j, k] = np.linalg.det(np.eye(3)[[i, j, k]])
    s = cross[0, 1, 2] / eps[0, 1, 2]
    assert abs(abs(s) - 1 / np.sqrt(2)) < 1e-12
    np.testing.assert_allclose(cross, s * eps, atol=1e-12)
    # parity rule: 1o x 1o cannot give 1o
    assert cue.O3.clebsch_gordan(one, one, one).shape[0] == 0
    # squared norm is 2 l3 + 1 in this normalisation
    for l1, l2, l3 in [(1, 1, 2), (2, 2, 2), (3, 2, 1), (3, 3, 0)]:
        c = cue.SO3.clebsch_gordan(cue.SO3(l1), cue.SO3(l2), cue.SO3(l3))
        assert abs((c**2).sum() - (2 * l3 + 1)) < 1e-10


def test_o3_order_and_selection_rule():
    names = ["0e", "0o", "1o", "1e", "2e", "2o", "3o", "3e"]
    irs = [cue.O3.from_string(n) for n in names]
    assert sorted(reversed(irs), key=lambda ir: ir._key()) == irs
    it = cue.O3.iterator()
    assert [repr(next(it)) for _ in range(6)] == ["0e", "0o", "1o", "1e", "2e", "2o"]
    assert [repr(r) for r in cue.O3(1, -1) * cue.O3(2, 1)] == ["1o", "2o", "3o"]
    assert cue.O3.trivial() == cue.O3(0, 1)


def test_irreps_container_documented_behaviour():
    assert repr(cue.Irreps("SO3", "16x0 + 4x1")) == "16x0+4x1"
    r = cue.Irreps("SO3", "1 + 2 + 0 + 1").sort()
    assert repr(r.irreps) == "0+1+1+2" and r.perm == (1, 3, 0, 2) and r.inv == (2, 0, 3, 1)
    assert repr(cue.Irreps("SO3", "1 + 2 + 0 + 1").regroup()) == "0+2x1+2"
    assert repr(cue.Irreps("SO3", "1 + 0x2 + 1").simplify()) == "2x1"
    assert cue.Irreps("SO3", "100x0 + 10x1").dim == 130
    assert cue.Irreps("SO3", "100x0 + 20x1 + 10x0").count("0") == 110
    assert repr(cue.Irreps("SO3", "32x1").new_scalars(2)) == "2x0"
    assert cue.Irreps("SO3", "100x0 + 10x1").slices() == [slice(0, 100), slice(100, 130)]
    assert repr(cue.Irreps("SO3", "4x0 + 4x1 + 2x2").filter(keep="0 + 1")) == "4x0+4x1"
    assert repr(cue.Irreps("SO3", "4x0 + 4x1 + 2x2").filter(drop="0 + 1")) == "2x2"
    assert repr(cue.Irreps("O3", "3x0e + 2x0e + 4x1o").set_mul(2)) == "2x0e+2x0e+2x1o"
    assert cue.Irreps("O3", "128x0e+128x1o+128x2e+128x3o").dim == 2048
    with pytest.raises(ValueError):
        cue.Irreps("O3", "3x1")
    assert cue.mul_ir.shape((32, cue.O3(2, -1))) == (32, 5) and cue.ir_mul.shape((32, cue.O3(2, -1))) == (5, 32)


def test_spherical_harmonics_values_norm_equivariance():
    sh = cue.descriptors.spherical_harmonics_values
    y = sh(cue.SO3(1), [0, 1, 2], np.array([0.0, 1.0, 0.0]))
    np.testing.assert_allclose(y, [1, 0, np.sqrt(3), 0, 0, 0, np.sqrt(5), 0, 0], atol=1e-12)
    rng = np.random.default_rng(0)
    v = rng.normal(size=(50, 3))
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    y = sh(cue.O3(1, -1), [0, 1, 2, 3], v)
    off = 0
    for ell in range(4):
        blk = y[:, off: off + 2 * ell + 1]
        np.testing.assert_allclose((blk**2).sum(1), 2 * ell + 1, atol=1e-10)
        off += 2 * ell + 1
    # homogeneity: Y_l(a x) = a^l Y_l(x)
    np.testing.assert_allclose(sh(cue.SO3(1), [3], 2.0 * v), 8.0 * sh(cue.SO3(1), [3], v), atol=1e-10)
    # equivariance under an infinitesimal rotation generated by X: d/dt Y_l(exp(tX1) x) = X_l Y_l(x)
    ell = 2
    X1, Xl = cue.SO3(1).X, cue.SO3(ell).X
    x = v[:5]
    h = 1e-6
    for gidx in range(3):
        xr = x + h * x @ X1[gidx].T
        xl = x - h * x @ X1[gidx].T
        num = (sh(cue.SO3(1), [ell], xr) - sh(cue.SO3(1), [ell], xl)) / (2 * h)
        ana = sh(cue.SO3(1), [ell], x) @ Xl[gidx].T
        np.testing.assert_allclose(num, ana, atol=1e-6)
