"""Irreducible representations of SU(2), SO(3), O(3) and direct sums of them.

Host-side mirror of the reference's group-theory layer, restricted to what the
segmented-polynomial hot path needs: parsing ``"128x0e+128x1o"``, the O3
ordering, the selection rule, real Clebsch-Gordan coefficients and the two
data layouts.

Reference behaviour followed (files relative to
``cuequivariance/cuequivariance/group_theory``):

* ``representations/irrep_su2.py:82-90,188-279``  SU(2) Clebsch-Gordan (Racah sum, exact fractions)
* ``representations/irrep_so3.py:29-41,81-96``    real basis change with the ``(-i)^l`` phase
* ``representations/irrep_o3.py:62-88``           parity rule, order key ``(l, -p*(-1)^l)``
* ``irreps_array/irreps.py:40-470``               ``Irreps`` container (``sort``, ``simplify``, ...)
* ``irreps_array/irreps_layout.py:23-89``         ``mul_ir`` / ``ir_mul``
"""

from __future__ import annotations

import dataclasses
import functools
import re
from enum import Enum
from fractions import Fraction
from math import factorial
from typing import Iterable, NamedTuple, Sequence, Union

import numpy as np

__all__ = [
    "Irrep",
    "SU2",
    "SO3",
    "O3",
    "MulIrrep",
    "Irreps",
    "IrrepsLayout",
    "mul_ir",
    "ir_mul",
    "IrrepsAndLayout",
    "clebsch_gordan",
    "into_list_of_irrep",
]


# --------------------------------------------------------------------------
# SU(2) Clebsch-Gordan coefficients, exact rational arithmetic under the root
# --------------------------------------------------------------------------
def _su2_cg_coeff(j1: Fraction, m1: Fraction, j2: Fraction, m2: Fraction, j3: Fraction, m3: Fraction) -> float:
    """<j1 m1 j2 m2 | j3 m3> * sqrt(2 j3 + 1) ... see note in :func:`su2_clebsch_gordan`.

    Racah's closed form evaluated with exact fractions; only the final square
    root is taken in floating point (reference ``irrep_su2.py:220-279``).
    """
    if m3 != m1 + m2:
        return 0.0
    vmin = int(max(-j1 + j2 + m3, -j1 + m1, 0))
    vmax = int(min(j2 + j3 + m1, j3 - j1 + j2, j3 + m3))

    def f(n) -> int:
        assert n == round(n)
        return factorial(round(n))

    pref = (2 * j3 + 1) * Fraction(
        f(j3 + j1 - j2) * f(j3 - j1 + j2) * f(j1 + j2 - j3) * f(j3 + m3) * f(j3 - m3),
        f(j1 + j2 + j3 + 1) * f(j1 - m1) * f(j1 + m1) * f(j2 - m2) * f(j2 + m2),
    )
    s = Fraction(0)
    for v in range(vmin, vmax + 1):
        s += (-1) ** int(v + j2 + m2) * Fraction(
            f(j2 + j3 + m1 - v) * f(j1 - m1 + v),
            f(v) * f(j3 - j1 + j2 - v) * f(j3 + m3 - v) * f(v + j1 - j2 - m3),
        )
    mag = float(pref * s * s) ** 0.5
    return mag if s > 0 else -mag


@functools.lru_cache(maxsize=None)
def _su2_cg_matrix(tj1: int, tj2: int, tj3: int) -> np.ndarray:
    """CG tensor ``[m1, m2, m3]`` for doubled spins ``tj = 2 j``.

    Normalisation: *not* divided by ``sqrt(2 j3 + 1)``, so for fixed ``m3`` the
    squares sum to one and the whole tensor has squared norm ``2 j3 + 1``
    (reference ``irrep_su2.py:188-217``).
    """
    d1, d2, d3 = tj1 + 1, tj2 + 1, tj3 + 1
    mat = np.zeros((d1, d2, d3), dtype=np.float64)
    if tj3 not in range(abs(tj1 - tj2), tj1 + tj2 + 1, 2):
        return mat
    j1, j2, j3 = Fraction(tj1, 2), Fraction(tj2, 2), Fraction(tj3, 2)
    for a in range(d1):
        m1 = -j1 + a
        for b in range(d2):
            m2 = -j2 + b
            m3 = m1 + m2
            if abs(m3) <= j3:
                mat[a, b, int(j3 + m3)] = _su2_cg_coeff(j1, m1, j2, m2, j3, m3)
    mat.setflags(write=False)
    return mat


def _su2_generators(tj: int) -> np.ndarray:
    """Lie-algebra generators of the spin-``tj/2`` representation (reference ``irrep_su2.py:111-127``)."""
    j = tj / 2
    m = np.arange(-j, j)
    raising = np.diag(-np.sqrt(j * (j + 1) - m * (m + 1)), k=-1)
    m = np.arange(-j + 1, j + 1)
    lowering = np.diag(np.sqrt(j * (j + 1) - m * (m - 1)), k=1)
    m = np.arange(-j, j + 1)
    return np.stack([0.5 * (raising + lowering), np.diag(1j * m), -0.5j * (raising - lowering)], axis=0)


def _real_to_complex(ell: int) -> np.ndarray:
    """Unitary change of basis from real to complex spherical harmonics of degree ``ell``.

    The extra ``(-i)^ell`` makes the transformed Clebsch-Gordan tensors real
    (reference ``irrep_so3.py:29-41``).
    """
    q = np.zeros((2 * ell + 1, 2 * ell + 1), dtype=np.complex128)
    s = 1 / np.sqrt(2)
    for m in range(-ell, 0):
        q[ell + m, ell + abs(m)] = s
        q[ell + m, ell - abs(m)] = -1j * s
    q[ell, ell] = 1
    for m in range(1, ell + 1):
        q[ell + m, ell + abs(m)] = (-1) ** m * s
        q[ell + m, ell - abs(m)] = 1j * (-1) ** m * s
    return q * (-1j) ** ell


@functools.lru_cache(maxsize=None)
def _so3_cg(l1: int, l2: int, l3: int) -> np.ndarray:
    """Real Clebsch-Gordan tensor of shape ``(npaths, 2l1+1, 2l2+1, 2l3+1)`` (reference ``irrep_so3.py:81-96``)."""
    if l3 not in range(abs(l1 - l2), l1 + l2 + 1):
        return np.zeros((0, 2 * l1 + 1, 2 * l2 + 1, 2 * l3 + 1))
    c = _su2_cg_matrix(2 * l1, 2 * l2, 2 * l3)[None]
    q1, q2, q3 = _real_to_complex(l1), _real_to_complex(l2), _real_to_complex(l3)
    c = np.einsum("ij,kl,mn,zikn->zjlm", q1, q2, np.conj(q3.T), c)
    assert np.all(np.abs(np.imag(c)) < 1e-5)
    c = np.ascontiguousarray(np.real(c))
    c.setflags(write=False)
    return c


# --------------------------------------------------------------------------
# Irrep classes
# --------------------------------------------------------------------------
class Irrep:
    """Base class: an irreducible representation with an order, a selection rule and CG coefficients."""

    @classmethod
    def regexp_pattern(cls) -> re.Pattern:
        raise NotImplementedError

    @classmethod
    def from_string(cls, s: str) -> "Irrep":
        raise NotImplementedError

    @classmethod
    def _from(cls, x) -> "Irrep":
        if isinstance(x, cls):
            return x
        if isinstance(x, str):
            return cls.from_string(x)
        if isinstance(x, MulIrrep):
            return cls._from(x.ir)
        if isinstance(x, tuple):
            return cls(*x)
        return cls(x)

    @classmethod
    def trivial(cls) -> "Irrep":
        for ir in cls.iterator():
            if ir.is_scalar():
                return ir
        raise ValueError("no trivial irrep")  # pragma: no cover

    def is_scalar(self) -> bool:
        raise NotImplementedError

    def is_trivial(self) -> bool:
        return self.is_scalar()

    @property
    def X(self):
        """Generators of the Lie algebra in this representation, shape ``(3, dim, dim)``."""
        return self.continuous_generators()

    def __le__(self, other) -> bool:
        return self == other or self < other


@dataclasses.dataclass(frozen=True)
class SU2(Irrep):
    """Spin-``j`` representation of SU(2); ``j`` may be a half-integer."""

    j: float

    @classmethod
    def regexp_pattern(cls) -> re.Pattern:
        return re.compile(r"(\d+(?:/2)?)")

    @classmethod
    def from_string(cls, s: str) -> "SU2":
        s = s.strip()
        return cls(j=int(s[:-2]) / 2) if s.endswith("/2") else cls(j=int(s))

    def __repr__(self) -> str:
        return f"{int(self.j)}" if round(self.j) == self.j else f"{int(2 * self.j)}/2"

    def __mul__(self, other) -> list["SU2"]:
        other = SU2._from(other)
        a, b = int(2 * self.j), int(2 * other.j)
        return [SU2(j=t / 2) for t in range(abs(a - b), a + b + 1, 2)]

    @classmethod
    def clebsch_gordan(cls, r1, r2, r3) -> np.ndarray:
        r1, r2, r3 = cls._from(r1), cls._from(r2), cls._from(r3)
        if r3 in r1 * r2:
            return np.array(_su2_cg_matrix(int(2 * r1.j), int(2 * r2.j), int(2 * r3.j)))[None]
        return np.zeros((0, r1.dim, r2.dim, r3.dim))

    @property
    def dim(self) -> int:
        return int(2 * self.j + 1)

    def is_scalar(self) -> bool:
        return self.j == 0

    def __lt__(self, other) -> bool:
        return self.j < SU2._from(other).j

    @classmethod
    def iterator(cls):
        t = 0
        while True:
            yield cls(j=t / 2)
            t += 1

    def continuous_generators(self) -> np.ndarray:
        return _su2_generators(int(2 * self.j))


@dataclasses.dataclass(frozen=True)
class SO3(Irrep):
    """Real degree-``l`` representation of SO(3)."""

    l: int  # noqa: E741

    @classmethod
    def regexp_pattern(cls) -> re.Pattern:
        return re.compile(r"(\d+)")

    @classmethod
    def from_string(cls, s: str) -> "SO3":
        return cls(l=int(s))

    def __repr__(self) -> str:
        return f"{self.l}"

    def __mul__(self, other) -> list["SO3"]:
        other = SO3._from(other)
        return [SO3(l=ell) for ell in range(abs(self.l - other.l), self.l + other.l + 1)]

    @classmethod
    def clebsch_gordan(cls, r1, r2, r3) -> np.ndarray:
        r1, r2, r3 = cls._from(r1), cls._from(r2), cls._from(r3)
        return np.array(_so3_cg(r1.l, r2.l, r3.l))

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def is_scalar(self) -> bool:
        return self.l == 0

    def __lt__(self, other) -> bool:
        return self.l < SO3._from(other).l

    @classmethod
    def iterator(cls):
        ell = 0
        while True:
            yield cls(l=ell)
            ell += 1

    def continuous_generators(self) -> np.ndarray:
        """Real antisymmetric generators ``X = Q^H X_su2 Q`` (reference ``irrep_so3.py:111-116``)."""
        x = _su2_generators(2 * self.l)
        q = _real_to_complex(self.l)
        x = np.conj(q.T) @ x @ q
        assert np.all(np.abs(np.imag(x)) < 1e-5)
        return np.real(x)


@dataclasses.dataclass(frozen=True)
class O3(Irrep):
    """Real representation of O(3): degree ``l`` and parity ``p`` (+1 even, -1 odd)."""

    l: int  # noqa: E741
    p: int

    @classmethod
    def regexp_pattern(cls) -> re.Pattern:
        return re.compile(r"(\d+)([eo])")

    @classmethod
    def from_string(cls, s: str) -> "O3":
        s = s.strip()
        return cls(l=int(s[:-1]), p={"e": 1, "o": -1}[s[-1]])

    def __repr__(self) -> str:
        return f"{self.l}{'o' if self.p < 0 else 'e'}"

    def __mul__(self, other) -> list["O3"]:
        other = O3._from(other)
        p = self.p * other.p
        return [O3(l=ell, p=p) for ell in range(abs(self.l - other.l), self.l + other.l + 1)]

    @classmethod
    def clebsch_gordan(cls, r1, r2, r3) -> np.ndarray:
        r1, r2, r3 = cls._from(r1), cls._from(r2), cls._from(r3)
        if r1.p * r2.p == r3.p:
            return np.array(_so3_cg(r1.l, r2.l, r3.l))
        return np.zeros((0, r1.dim, r2.dim, r3.dim))

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def is_scalar(self) -> bool:
        return self.l == 0 and self.p == 1

    def _key(self):
        # 0e < 0o < 1o < 1e < 2e < 2o < ...   (reference irrep_o3.py:86-88)
        return (self.l, -self.p * (-1) ** self.l)

    def __lt__(self, other) -> bool:
        return self._key() < O3._from(other)._key()

    @classmethod
    def iterator(cls):
        ell = 0
        while True:
            yield cls(l=ell, p=(-1) ** ell)
            yield cls(l=ell, p=-((-1) ** ell))
            ell += 1

    def continuous_generators(self) -> np.ndarray:
        return SO3(l=self.l).continuous_generators()


class O3_e3nn(O3):
    """O(3) irreps ordered the e3nn way, ``(l, p)`` ascending: ``0e < 0o < 1e < 1o < ...`` (reference
    ``group_theory/experimental/e3nn.py:23-52``).  The reference takes the coefficients of this group from
    ``e3nn.o3.wigner_3j(l1, l2, l3) * sqrt(2 l3 + 1)``; they are the same real-basis tensors as :class:`O3`'s
    (same ``(-i)^l`` change of basis, same normalisation), which is what is used here."""

    def __mul__(self, other) -> list["O3_e3nn"]:
        return [O3_e3nn(l=ir.l, p=ir.p) for ir in O3.__mul__(self, other)]

    def _key(self):
        return (self.l, self.p)

    def __lt__(self, other) -> bool:
        return self._key() < O3_e3nn._from(other)._key()

    @classmethod
    def iterator(cls):
        ell = 0
        while True:
            yield cls(l=ell, p=(-1) ** ell)
            yield cls(l=ell, p=-((-1) ** ell))
            ell += 1


_IRREP_CLASSES = {"SU2": SU2, "SO3": SO3, "O3": O3}


def clebsch_gordan(r1: Irrep, r2: Irrep, r3: Irrep) -> np.ndarray:
    """CG tensor of shape ``(number_of_paths, r1.dim, r2.dim, r3.dim)``."""
    return type(r1).clebsch_gordan(r1, r2, r3)


# --------------------------------------------------------------------------
# Irreps container
# --------------------------------------------------------------------------
# ---- assumed irrep class and layout (reference: irreps_array/context_irrep_class.py, context_layout.py, context_decorator.py) ----
_assumed = {"irrep_class": None, "layout": None}


def get_irrep_scope(raising: bool = True):
    """The irrep class assumed by the enclosing ``with cue.assume(...)`` (a name such as ``"O3"`` is looked up)."""
    value = _assumed["irrep_class"]
    if raising and value is None:
        raise ValueError("No irrep class set in the context. Please specify the irrep class explicitly or use ``with cue.assume(irrep):``.")
    return _IRREP_CLASSES[value] if isinstance(value, str) else value


def get_layout_scope(raising: bool = True):
    """The layout assumed by the enclosing ``with cue.assume(...)``."""
    value = _assumed["layout"]
    if raising and value is None:
        raise ValueError("No layout set in the context. Please specify the layout explicitly or use ``with cue.assume(layout):``.")
    return value


class assume:
    """Context manager and decorator: inside, ``cue.Irreps("2x1")`` takes the given irrep class and a layout left out (``None``)
    is the given one.  ``cue.assume(cue.SO3, cue.ir_mul)``, ``cue.assume("O3")``, ``cue.assume(cue.mul_ir)``."""

    def __init__(self, irrep_class=None, layout=None):
        if isinstance(irrep_class, IrrepsLayout) and layout is None:
            irrep_class, layout = None, irrep_class
        self.irrep_class, self.layout = irrep_class, layout

    def __enter__(self):
        self._before = dict(_assumed)
        _assumed["irrep_class"], _assumed["layout"] = self.irrep_class, self.layout
        return self

    def __exit__(self, *exc):
        _assumed.update(self._before)
        return False

    def __call__(self, func):
        @functools.wraps(func)
        def wrapper(*args, **kwargs):
            with self:
                return func(*args, **kwargs)

        return wrapper


@dataclasses.dataclass(frozen=True)
class MulIrrep:
    mul: int
    ir: Irrep

    def __repr__(self) -> str:
        return f"{self.ir}" if self.mul == 1 else f"{self.mul}x{self.ir}"

    def __iter__(self):
        return iter((self.mul, self.ir))

    @property
    def dim(self) -> int:
        return self.mul * self.ir.dim


class SortResult(NamedTuple):
    irreps: "Irreps"
    perm: tuple
    inv: tuple


class Irreps:
    """Direct sum of irreps with multiplicities, e.g. ``Irreps("O3", "128x0e + 128x1o")``."""

    __slots__ = ("irrep_class", "_mulirreps")

    def __init__(self, *args):
        if len(args) == 1 and isinstance(args[0], Irreps):
            args = (args[0].irrep_class, args[0]._mulirreps)
        elif len(args) == 1 and isinstance(args[0], Irrep):
            args = (type(args[0]), [(1, args[0])])
        elif len(args) == 1:
            # Without an explicit group: the one assumed by the enclosing ``with cue.assume(...)``, else the string decides
            # ("0e" / "1o" is O3, bare integers SO3).
            text = args[0]
            scope = get_irrep_scope(raising=False)
            if scope is not None:
                args = (scope, text)
            elif isinstance(text, str):
                args = (O3 if re.search(r"\d[eo]", text) else SO3, text)
            else:
                raise ValueError("Irreps needs an irrep class")
        if len(args) != 2:
            raise ValueError(f"Irreps requires (irrep_class, input); got {len(args)} arguments")
        irrep_class, inp = args
        if isinstance(irrep_class, str):
            irrep_class = _IRREP_CLASSES[irrep_class]
        elif isinstance(irrep_class, Irreps):
            irrep_class = irrep_class.irrep_class
        elif isinstance(irrep_class, Irrep):
            irrep_class = type(irrep_class)
        assert isinstance(irrep_class, type) and issubclass(irrep_class, Irrep)

        out = []
        if isinstance(inp, str):
            for term in [] if inp.strip() == "" else inp.split("+"):
                if "x" in term:
                    mul, rep = term.split("x")
                    mul, rep = int(mul), rep.strip()
                else:
                    mul, rep = 1, term.strip()
                if not re.fullmatch(irrep_class.regexp_pattern(), rep):
                    raise ValueError(
                        f"Invalid representation string: {rep}, expected pattern: {irrep_class.regexp_pattern().pattern}"
                    )
                out.append(MulIrrep(mul, irrep_class.from_string(rep)))
        elif isinstance(inp, Irreps):
            if inp.irrep_class is not irrep_class:
                raise ValueError(f"Invalid representation: {inp.irrep_class}, expected {irrep_class}")
            out = list(inp._mulirreps)
        else:
            for x in inp:
                if isinstance(x, MulIrrep):
                    if not isinstance(x.ir, irrep_class):
                        raise ValueError(f"Invalid representation: {x.ir}, expected {irrep_class}")
                    out.append(x)
                elif isinstance(x, irrep_class):
                    out.append(MulIrrep(1, x))
                else:
                    try:
                        mul, ir = x
                    except (ValueError, TypeError):
                        raise ValueError(f"Invalid representation: {x}, expected (mul, irrep)")
                    if not isinstance(mul, (int, np.integer)):
                        raise ValueError(f"Invalid multiplicity: {mul}, expected int")
                    out.append(MulIrrep(int(mul), irrep_class._from(ir)))
        object.__setattr__(self, "irrep_class", irrep_class)
        object.__setattr__(self, "_mulirreps", tuple(out))

    def __setattr__(self, *a):  # immutable
        raise AttributeError("Irreps is immutable")

    # immutable value: copies are the object itself, pickles rebuild it from its parts
    def __copy__(self):
        return self

    def __deepcopy__(self, memo):
        return self

    def __reduce__(self):
        return (Irreps, (self.irrep_class, self._mulirreps))

    def __len__(self):
        return len(self._mulirreps)

    def __iter__(self):
        return iter(self._mulirreps)

    def __getitem__(self, i):
        x = self._mulirreps[i]
        return Irreps(self.irrep_class, x) if isinstance(i, slice) else x

    def __contains__(self, rep) -> bool:
        rep = self.irrep_class._from(rep)
        return any(m.ir == rep for m in self)

    def __repr__(self):
        return "+".join(f"{m}" for m in self)

    def __hash__(self):
        return hash((self.irrep_class, self._mulirreps))

    def __eq__(self, other):
        try:
            other = Irreps(self.irrep_class, other)
        except (ValueError, KeyError, TypeError, AssertionError):
            return False
        return self.irrep_class is other.irrep_class and self._mulirreps == other._mulirreps

    def __add__(self, other):
        other = Irreps(self.irrep_class, other)
        return Irreps(self.irrep_class, self._mulirreps + other._mulirreps)

    def __radd__(self, other):
        return Irreps(self.irrep_class, other) + self

    def __mul__(self, k):
        if isinstance(k, int):
            return Irreps(self.irrep_class, [MulIrrep(m * k, ir) for m, ir in self])
        return NotImplemented

    __rmul__ = __mul__

    def __floordiv__(self, k):
        if isinstance(k, int):
            return Irreps(self.irrep_class, [MulIrrep(m // k, ir) for m, ir in self])
        return NotImplemented

    def new_scalars(self, mul: int) -> "Irreps":
        return Irreps(self.irrep_class, [(mul, self.irrep_class.trivial())])

    def count(self, rep) -> int:
        rep = self.irrep_class._from(rep)
        return sum(m for m, ir in self if ir == rep)

    @property
    def dim(self) -> int:
        return sum(m * ir.dim for m, ir in self)

    @property
    def num_irreps(self) -> int:
        return sum(m for m, _ in self)

    @property
    def muls(self) -> list[int]:
        return [m for m, _ in self]

    def slices(self) -> list[slice]:
        out, i = [], 0
        for m, ir in self:
            out.append(slice(i, i + m * ir.dim))
            i += m * ir.dim
        return out

    def is_scalar(self) -> bool:
        return all(ir.is_scalar() for _, ir in self)

    def merge_consecutive(self) -> "Irreps":
        out = []
        for m, ir in self:
            if out and out[-1][1] == ir:
                out[-1] = (out[-1][0] + m, ir)
            else:
                out.append((m, ir))
        return Irreps(self.irrep_class, out)

    def remove_zero_multiplicities(self) -> "Irreps":
        return Irreps(self.irrep_class, [(m, ir) for m, ir in self if m != 0])

    def simplify(self) -> "Irreps":
        return self.remove_zero_multiplicities().merge_consecutive()

    def sort(self) -> SortResult:
        """Stable sort by ``(irrep, original position)``; ``inv[new] = old`` and ``perm[old] = new``."""
        order = sorted(range(len(self)), key=lambda i: (_OrderKey(self[i].ir), i))
        inv = tuple(order)
        perm = tuple(inv.index(i) for i in range(len(inv)))
        return SortResult(Irreps(self.irrep_class, [self[i] for i in order]), perm, inv)

    def regroup(self) -> "Irreps":
        return self.sort().irreps.simplify()

    def set_mul(self, mul: int) -> "Irreps":
        return Irreps(self.irrep_class, [(mul, ir) for _, ir in self])

    def filter(self, *, keep=None, drop=None) -> "Irreps":
        if (keep is None) == (drop is None):
            raise ValueError("exactly one of keep / drop must be given")
        if keep is not None:
            pred = keep if callable(keep) else (lambda m, s=into_list_of_irrep(self.irrep_class, keep): m.ir in s)
        else:
            pred = (
                (lambda m: not drop(m))
                if callable(drop)
                else (lambda m, s=into_list_of_irrep(self.irrep_class, drop): m.ir not in s)
            )
        return Irreps(self.irrep_class, [m for m in self if pred(m)])

    def layout_insensitive(self) -> bool:
        return all(not (m > 1 and ir.dim > 1) for m, ir in self)


@functools.total_ordering
class _OrderKey:
    """Adapter so that ``sorted`` uses the irrep's own ``__lt__``."""

    __slots__ = ("ir",)

    def __init__(self, ir):
        self.ir = ir

    def __eq__(self, o):
        return self.ir == o.ir

    def __lt__(self, o):
        return self.ir < o.ir


def into_list_of_irrep(irrep_class, inp) -> list[Irrep]:
    """Accept a string, an irrep, a MulIrrep or an iterable of those (reference ``irrep_utils.py:21-50``)."""
    if isinstance(inp, str):
        return [ir for _, ir in Irreps(irrep_class, inp)]
    if isinstance(inp, Irrep):
        return [inp]
    if isinstance(inp, MulIrrep):
        return [inp.ir]
    try:
        it = iter(inp)
    except TypeError:
        return [irrep_class._from(inp)]
    out = []
    for r in it:
        if isinstance(r, Irrep):
            out.append(r)
        elif isinstance(r, MulIrrep):
            out.append(r.ir)
        else:
            out.append(irrep_class._from(r))
    return out


# --------------------------------------------------------------------------
# Layouts
# --------------------------------------------------------------------------
class IrrepsLayout(Enum):
    """``mul_ir``: (multiplicity, component) as in e3nn. ``ir_mul``: (component, multiplicity), channels contiguous."""

    mul_ir = 1
    ir_mul = 2

    def shape(self, mulir) -> tuple[int, int]:
        mul, ir = mulir
        return (mul, ir.dim) if self is IrrepsLayout.mul_ir else (ir.dim, mul)

    def __repr__(self) -> str:
        return "(mul,irrep)" if self is IrrepsLayout.mul_ir else "(irrep,mul)"

    __str__ = __repr__

    @staticmethod
    def as_layout(layout) -> "IrrepsLayout":
        if isinstance(layout, IrrepsLayout):
            return layout
        if layout is None:  # the layout assumed by the enclosing ``with cue.assume(...)``, else the e3nn layout
            scope = get_layout_scope(raising=False)
            return IrrepsLayout.mul_ir if scope is None else scope
        try:
            return IrrepsLayout[layout]
        except KeyError:
            raise ValueError(f"Invalid layout {layout}")


mul_ir = IrrepsLayout.mul_ir
ir_mul = IrrepsLayout.ir_mul


@dataclasses.dataclass(frozen=True)
class IrrepsAndLayout:
    """A representation given as irreps plus the memory layout of each ``mul x ir`` block."""

    irreps: Irreps
    layout: IrrepsLayout

    def __init__(self, irreps, layout=None):
        object.__setattr__(self, "irreps", Irreps(irreps))
        object.__setattr__(self, "layout", IrrepsLayout.as_layout(layout))

    @property
    def dim(self) -> int:
        return self.irreps.dim

    def __repr__(self):
        return f"{self.irreps}"
