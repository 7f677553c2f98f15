"""Segmented tensor product descriptor: operands made of segments, paths with coefficients.

An operand is a flat vector cut into *segments*, each segment a small tensor whose
axes are named by one letter ("modes").  A *path* picks one segment per operand
and carries a coefficient array; the descriptor stands for

    last_operand[seg] += einsum(coeff, operand_0[seg_0], operand_1[seg_1], ...)

summed over paths.  This module is the host-side mirror of the reference's
descriptor IR, restricted to the transformations the executor needs.

Reference behaviour followed (``cuequivariance/cuequivariance/segmented_polynomials``):

* ``segmented_tensor_product.py:658-784``   add_path / insert_path (segments created on the fly)
* ``segmented_tensor_product.py:1045-1069`` permute_segments (paths keep their order)
* ``segmented_tensor_product.py:1098-1152`` squeeze_modes
* ``segmented_tensor_product.py:1154-1234`` split_mode
* ``segmented_tensor_product.py:1243-1284`` normalize_paths_for_operand
* ``segmented_tensor_product.py:1310-1332`` consolidate_paths
* ``segmented_tensor_product.py:1334-1427`` sort_indices_for_identical_operands / symmetrize_operands
* ``segmented_tensor_product.py:1472-1637`` flatten_modes / flatten_coefficient_modes (order of emitted paths)
* ``segmented_operand.py:23-233``, ``path.py:32-121``, ``subscripts.py:23-356``
"""

from __future__ import annotations

import base64
import itertools
import json
import math
import re
import zlib
from typing import Optional, Sequence, Union

import numpy as np

__all__ = ["Subscripts", "SegmentedOperand", "Path", "SegmentedTensorProduct"]


class Subscripts(str):
    """``"uv,iu,jv,kuv+ijk"``: comma (or underscore) separated operand modes, coefficient modes after ``+``."""

    def __new__(cls, s):
        if not isinstance(s, str):
            s = ",".join(s)
        s = s.replace("_", ",")
        if not cls.is_valid(s):
            raise ValueError(f"invalid subscripts {s}.")
        return super().__new__(cls, s)

    @staticmethod
    def is_valid(s) -> bool:
        if not isinstance(s, str):
            return False
        if re.match(r"^[a-z*]*(,[a-z*]*)*(\+[a-z*]*)?$", s) is None:
            return False
        return all(len(set(x)) == len(x) for x in re.split(r"[,+]", s))

    @classmethod
    def from_operands(cls, operands: Sequence[str], coefficients: str = "") -> "Subscripts":
        s = ",".join(operands)
        return cls(s + "+" + coefficients) if coefficients else cls(s)

    @property
    def operands(self) -> tuple[str, ...]:
        return tuple(self.split("+")[0].split(","))

    @property
    def coefficients(self) -> str:
        return self.split("+")[1] if "+" in self else ""

    @property
    def num_operands(self) -> int:
        return len(self.operands)

    def modes(self) -> list[str]:
        out = []
        for ch in self:
            if ch.isalpha() and ch not in out:
                out.append(ch)
        return out


class SegmentedOperand:
    """List of segment shapes; all segments have ``ndim`` axes."""

    __slots__ = ("ndim", "segments")

    def __init__(self, segments=None, *, ndim: Optional[int] = None):
        segments = tuple(tuple(int(d) for d in s) for s in (segments or ()))
        if ndim is None:
            assert len(segments) > 0
            ndim = len(segments[0])
        assert all(len(s) == ndim for s in segments)
        self.ndim = int(ndim)
        self.segments = segments

    @classmethod
    def empty_segments(cls, num_segments: int) -> "SegmentedOperand":
        return cls([()] * num_segments, ndim=0)

    def copy(self) -> "SegmentedOperand":
        return SegmentedOperand(self.segments, ndim=self.ndim)

    def with_segments(self, segments) -> "SegmentedOperand":
        return SegmentedOperand(segments, ndim=self.ndim)

    def __hash__(self):
        return hash((self.ndim, self.segments))

    def __eq__(self, o):
        return isinstance(o, SegmentedOperand) and self.ndim == o.ndim and self.segments == o.segments

    def __lt__(self, o):
        return (self.ndim, self.segments) < (o.ndim, o.segments)

    def __repr__(self):
        return f"Operand(ndim={self.ndim} num_segments={self.num_segments} size={self.size})"

    def __getitem__(self, i):
        return self.segments[i]

    def __len__(self):
        return len(self.segments)

    def __iter__(self):
        return iter(self.segments)

    @property
    def num_segments(self) -> int:
        return len(self.segments)

    @property
    def size(self) -> int:
        return sum(math.prod(s) for s in self.segments)

    def segment_offsets(self) -> list[int]:
        out, off = [], 0
        for s in self.segments:
            out.append(off)
            off += math.prod(s)
        return out

    def segment_slices(self) -> list[slice]:
        return [slice(o, o + math.prod(s)) for o, s in zip(self.segment_offsets(), self.segments)]

    def get_dims(self, axis: int) -> set[int]:
        return {s[axis] for s in self.segments}

    def all_same_segment_shape(self) -> bool:
        """False when there is no segment at all (same convention as the reference)."""
        return self.num_segments > 0 and len(set(self.segments)) == 1

    @property
    def segment_shape(self) -> tuple[int, ...]:
        if not self.all_same_segment_shape():
            raise ValueError("Segments do not have the same shape.")
        return self.segments[0]

    @property
    def segment_size(self) -> int:
        return math.prod(self.segment_shape)

    def squeeze(self) -> "SegmentedOperand":
        keep = [i for i in range(self.ndim) if self.get_dims(i) != {1}]
        if len(keep) == self.ndim:
            return self
        return SegmentedOperand([tuple(s[i] for i in keep) for s in self.segments], ndim=len(keep))


class Path:
    """One segment index per operand plus a float64 coefficient array."""

    __slots__ = ("indices", "coefficients")

    def __init__(self, indices, coefficients):
        self.indices = tuple(int(i) for i in indices)
        c = np.array(coefficients, dtype=np.float64)
        c.setflags(write=False)
        self.coefficients = c

    def __repr__(self):
        return f"Path({self.indices}, c.shape={self.coefficients.shape})"

    def __hash__(self):
        return hash((self.indices, self.coefficients.tobytes()))

    def __eq__(self, o):
        return self.indices == o.indices and np.array_equal(self.coefficients, o.coefficients)

    def __lt__(self, o):
        k1, k2 = (self.indices, self.coefficients.shape), (o.indices, o.coefficients.shape)
        if k1 != k2:
            return k1 < k2
        return tuple(self.coefficients.ravel()) < tuple(o.coefficients.ravel())

    def permute_operands(self, perm) -> "Path":
        return Path([self.indices[i] for i in perm], self.coefficients)


def _format_dims(dims: dict) -> str:
    def fmt(dd):
        if len(dd) == 0:
            return ""
        if len(dd) == 1:
            return str(next(iter(dd)))
        return "{" + ", ".join(str(i) for i in sorted(dd)) + "}"

    return " ".join(f"{m}={fmt(dd)}" for m, dd in sorted(dims.items()))


def _canon(i: int, n: int, what: str) -> int:
    if not -n <= i < n:
        raise ValueError(f"{what} {i} out of range [-{n}, {n})")
    return i % n if n else 0


class SegmentedTensorProduct:
    """Descriptor of a segmented tensor product (see module docstring)."""

    def __init__(self, operands_and_subscripts=None, coefficient_subscripts: str = "", *, paths=None):
        pairs = []
        for ope, ss in operands_and_subscripts or []:
            ope = ope.copy() if ope is not None else SegmentedOperand(ndim=len(ss))
            assert ope.ndim == len(ss)
            pairs.append([ope, str(ss)])
        self._ops: list[list] = pairs
        self.coefficient_subscripts = str(coefficient_subscripts)
        self.paths: tuple[Path, ...] = tuple(paths or ())

    # ---------------------------------------------------------------- construction
    @classmethod
    def from_subscripts(cls, subscripts) -> "SegmentedTensorProduct":
        s = Subscripts(subscripts)
        return cls([(None, ss) for ss in s.operands], s.coefficients)

    @classmethod
    def empty_segments(cls, num_segments: Sequence[int]) -> "SegmentedTensorProduct":
        """Descriptor whose operands are ``num_segments[k]`` scalar segments each, no paths yet."""
        return cls([(SegmentedOperand.empty_segments(n), "") for n in num_segments], "")

    @classmethod
    def from_dict(cls, data: dict) -> "SegmentedTensorProduct":
        d = cls.from_subscripts(data["subscripts"])
        for oid, ope in enumerate(data["operands"]):
            for seg in ope["segments"]:
                d.add_segment(oid, tuple(seg))
        for idx, c in zip(data["paths"]["indices"], data["paths"]["coefficients"]):
            d.add_path(*idx, c=np.array(c))
        return d

    @classmethod
    def from_json(cls, s: str):
        return cls.from_dict(json.loads(s))

    @classmethod
    def from_bytes(cls, b: bytes):
        return cls.from_json(zlib.decompress(b).decode("ascii"))

    @classmethod
    def from_base64(cls, s: str):
        return cls.from_bytes(base64.b64decode(s))

    def to_dict(self) -> dict:
        return {
            "subscripts": str(self.subscripts),
            "operands": [{"segments": [list(s) for s in o.segments]} for o in self.operands],
            "paths": {
                "indices": [list(p.indices) for p in self.paths],
                "coefficients": [p.coefficients.tolist() for p in self.paths],
            },
        }

    def to_json(self) -> str:
        return json.dumps(self.to_dict())

    def to_bytes(self) -> bytes:
        return zlib.compress(self.to_json().encode("ascii"))

    def to_base64(self) -> str:
        return base64.b64encode(self.to_bytes()).decode("ascii")

    def copy(self) -> "SegmentedTensorProduct":
        return SegmentedTensorProduct(self.operands_and_subscripts, self.coefficient_subscripts, paths=self.paths)

    def _replace(self, *, operands_and_subscripts=None, paths=None, coefficient_subscripts=None):
        return SegmentedTensorProduct(
            self.operands_and_subscripts if operands_and_subscripts is None else operands_and_subscripts,
            self.coefficient_subscripts if coefficient_subscripts is None else coefficient_subscripts,
            paths=self.paths if paths is None else paths,
        )

    # ---------------------------------------------------------------- properties
    @property
    def operands_and_subscripts(self) -> tuple:
        return tuple((o, s) for o, s in self._ops)

    @property
    def operands(self) -> tuple[SegmentedOperand, ...]:
        return tuple(o for o, _ in self._ops)

    @property
    def num_operands(self) -> int:
        return len(self._ops)

    @property
    def num_paths(self) -> int:
        return len(self.paths)

    @property
    def subscripts(self) -> Subscripts:
        return Subscripts.from_operands([s for _, s in self._ops], self.coefficient_subscripts)

    @property
    def indices(self) -> np.ndarray:
        if not self.paths:
            return np.empty((0, self.num_operands), dtype=int)
        return np.array([p.indices for p in self.paths], dtype=int)

    @property
    def stacked_coefficients(self) -> np.ndarray:
        return np.stack([p.coefficients for p in self.paths]) if self.paths else np.empty((0,))

    def __hash__(self):
        return hash((self.operands_and_subscripts, self.paths, self.coefficient_subscripts))

    def __eq__(self, o):
        if not isinstance(o, SegmentedTensorProduct):
            return NotImplemented
        return (
            self.operands_and_subscripts == o.operands_and_subscripts
            and self.paths == o.paths
            and self.coefficient_subscripts == o.coefficient_subscripts
        )

    def __lt__(self, o):
        a = (self.num_operands, self.num_paths, self.subscripts, self.operands, self.paths)
        b = (o.num_operands, o.num_paths, o.subscripts, o.operands, o.paths)
        return a < b

    def __repr__(self):
        sizes = ",".join(str(o.size) for o in self.operands)
        nseg = ",".join(str(len(o)) for o in self.operands)
        dims = _format_dims(self.get_dimensions_dict())
        return f"{self.subscripts} sizes={sizes} num_segments={nseg} num_paths={self.num_paths}" + (
            f" {dims}" if dims else ""
        )

    def to_text(self, coefficient_formatter=lambda x: f"{x}") -> str:
        """Multi-line dump: header, per-operand mode extents, memory cost, path indices and coefficients.

        Same layout as the reference's ``to_text`` except that the ``Flop cost`` line is omitted.
        """
        out = f"{self}"
        dims = self.get_dimensions_dict()
        for oid, (ope, ss) in enumerate(self.operands_and_subscripts):
            out += f"\noperand #{oid} subscripts={ss}"
            for i, ch in enumerate(ss):
                if len(dims[ch]) == 1:
                    out += f"\n  | {ch}: [{ope.segments[0][i]}] * {len(ope.segments)}"
                else:
                    out += f"\n  | {ch}: [" + ", ".join(str(s[i]) for s in ope.segments) + "]"
        out += f"\nMemory cost: {sum(o.size for o in self.operands)}"
        if self.paths:
            out += "\nPath indices: " + ", ".join(" ".join(str(i) for i in row) for row in self.indices)
            if all(len(dims[ch]) == 1 for ch in self.coefficient_subscripts):
                out += "\nPath coefficients: " + np.array2string(
                    self.stacked_coefficients, max_line_width=np.inf, formatter={"float": coefficient_formatter},
                    threshold=np.inf,
                )
            else:
                out += "\nPath coefficients:\n" + "\n".join(
                    np.array2string(p.coefficients, formatter={"float": coefficient_formatter}, threshold=np.inf)
                    for p in self.paths
                )
        else:
            out += "\nNo paths."
        return out

    def get_dimensions_dict(self) -> dict[str, set[int]]:
        dims = {m: set() for m in self.subscripts.modes()}
        for ope, ss in self._ops:
            for i, m in enumerate(ss):
                dims[m].update(ope.get_dims(i))
        return dims

    def get_dims(self, m: str) -> set[int]:
        return self.get_dimensions_dict().get(m, set())

    def get_path_dimensions_dict(self, path, *, returns_sets: bool = False) -> dict:
        if isinstance(path, int):
            path = self.paths[path]
        dims = {m: {d} for m, d in zip(self.coefficient_subscripts, path.coefficients.shape)}
        for oid, sid in enumerate(path.indices):
            for m, d in zip(self._ops[oid][1], self._ops[oid][0][sid]):
                dims.setdefault(m, set()).add(d)
        if returns_sets:
            return dims
        assert all(len(dd) == 1 for dd in dims.values())
        return {m: next(iter(dd)) for m, dd in dims.items()}

    def get_segment_shape(self, operand: int, path) -> tuple[int, ...]:
        if isinstance(path, int):
            path = self.paths[path]
        return self._ops[operand][0][path.indices[operand]]

    def all_same_segment_shape(self) -> bool:
        return all(o.all_same_segment_shape() for o in self.operands)

    def all_segments_are_used(self) -> bool:
        return all(
            any(s == p.indices[o] for p in self.paths)
            for o, ope in enumerate(self.operands)
            for s in range(ope.num_segments)
        )

    def assert_valid(self):
        for m in self.subscripts.modes():
            if self.subscripts.count(m) == 1:
                raise ValueError(f"mode {m} is not contracted in {self.subscripts}.")
        for p in self.paths:
            if p.coefficients.ndim != len(self.coefficient_subscripts):
                raise ValueError("coefficient rank mismatch")
            for oid, sid in enumerate(p.indices):
                if not 0 <= sid < self.operands[oid].num_segments:
                    raise ValueError(f"path index {sid} out of bounds for operand {oid}")
            if any(len(dd) != 1 for dd in self.get_path_dimensions_dict(p, returns_sets=True).values()):
                raise ValueError("path has ambiguous dimensions")

    # ---------------------------------------------------------------- builders (in place)
    def add_segment(self, operand: int, segment) -> int:
        if isinstance(segment, dict):
            segment = tuple(segment[m] for m in self._ops[operand][1])
        ope = self._ops[operand][0]
        if len(segment) != ope.ndim:
            raise ValueError(f"segment has {len(segment)} dimensions, expected {ope.ndim}.")
        self._ops[operand][0] = ope.with_segments(ope.segments + (tuple(segment),))
        return ope.num_segments

    def add_segments(self, operand: int, segments):
        for s in segments:
            self.add_segment(operand, s)

    def insert_segments(self, operand: int, sid: int, segments):
        """Insert segments before position ``sid`` (negative counts from one past the end) and shift path indices."""
        operand = _canon(operand, self.num_operands, "operand")
        n_old = self.operands[operand].num_segments
        sid = _canon(sid, n_old + 1, "sid")
        segments = [tuple(s) for s in segments]
        ope = self._ops[operand][0]
        self._ops[operand][0] = ope.with_segments(ope.segments[:sid] + tuple(segments) + ope.segments[sid:])
        k = len(segments)
        self.paths = tuple(
            Path([s if (o != operand or s < sid) else s + k for o, s in enumerate(p.indices)], p.coefficients)
            for p in self.paths
        )

    def insert_path(self, path_index: int, *segments, c, dims: Optional[dict] = None) -> int:
        """``segments[k]`` is a segment index, a shape, a ``{mode: extent}`` dict, or ``None`` (create a segment)."""
        path_index = _canon(path_index, len(self.paths) + 1, "path_index")
        if len(segments) != self.num_operands:
            raise ValueError(f"expected {self.num_operands} indices, got {len(segments)}.")
        coeff = np.asarray(c, dtype=np.float64)
        if coeff.ndim != len(self.coefficient_subscripts):
            raise ValueError(
                f"expected {len(self.coefficient_subscripts)} dimensions for the coefficients, got {coeff.ndim}."
            )
        modes = self.subscripts.modes()
        known: dict[str, set[int]] = {m: {d} for m, d in (dims or {}).items() if m in modes}
        for m, d in zip(self.coefficient_subscripts, coeff.shape):
            known.setdefault(m, set()).add(d)
        for oid, s in enumerate(segments):
            ss = self._ops[oid][1]
            if isinstance(s, (int, np.integer)):
                n = self.operands[oid].num_segments
                if not -n <= s < n:
                    raise ValueError(f"segment index {s} out of bounds for operand {oid}.")
                for m, d in zip(ss, self.operands[oid][s]):
                    known.setdefault(m, set()).add(d)
            elif isinstance(s, tuple):
                for m, d in zip(ss, s):
                    known.setdefault(m, set()).add(d)
            elif isinstance(s, dict):
                for m, d in s.items():
                    known.setdefault(m, set()).add(d)
            elif s is not None:
                raise ValueError(f"expected a segment index, a tuple or a dictionary. Got {s}.")
        if any(len(dd) != 1 for dd in known.values()):
            raise ValueError(f"Ambiguous dimensions for the path. {known}")
        if len(known) != len(modes):
            raise ValueError(f"missing dimensions for {set(modes) - known.keys()}.")
        ext = {m: next(iter(dd)) for m, dd in known.items()}
        idx = []
        for oid, s in enumerate(segments):
            if isinstance(s, (int, np.integer)):
                idx.append(int(s) % self.operands[oid].num_segments)
            else:
                idx.append(self.add_segment(oid, ext))
        paths = list(self.paths)
        paths.insert(path_index, Path(idx, coeff))
        self.paths = tuple(paths)
        return path_index

    def add_path(self, *segments, c, dims: Optional[dict] = None) -> int:
        return self.insert_path(len(self.paths), *segments, c=c, dims=dims)

    # ---------------------------------------------------------------- functional transforms
    def permute_operands(self, perm) -> "SegmentedTensorProduct":
        return self._replace(
            operands_and_subscripts=[self.operands_and_subscripts[i] for i in perm],
            paths=[p.permute_operands(perm) for p in self.paths],
        )

    def move_operand(self, operand: int, new_index: int) -> "SegmentedTensorProduct":
        operand = _canon(operand, self.num_operands, "operand")
        if new_index < 0:
            new_index += self.num_operands
        perm = list(range(self.num_operands))
        del perm[operand]
        perm.insert(new_index, operand)
        return self.permute_operands(perm)

    def move_operand_first(self, operand: int):
        return self.move_operand(operand, 0)

    def move_operand_last(self, operand: int):
        return self.move_operand(operand, -1)

    def permute_segments(self, operand: int, perm) -> "SegmentedTensorProduct":
        """New segment ``n`` is old segment ``perm[n]``; paths are relabelled, their order is kept."""
        operand = _canon(operand, self.num_operands, "operand")
        perm = list(perm)
        where = {old: new for new, old in enumerate(perm)}
        ops = list(self.operands_and_subscripts)
        ope, ss = ops[operand]
        ops[operand] = (ope.with_segments([ope[i] for i in perm]), ss)
        paths = [
            Path([s if o != operand else where[s] for o, s in enumerate(p.indices)], p.coefficients)
            for p in self.paths
        ]
        return self._replace(operands_and_subscripts=ops, paths=paths)

    def sort_paths(self, operands_ordering=None) -> "SegmentedTensorProduct":
        if operands_ordering is None:
            operands_ordering = range(self.num_operands)
        if isinstance(operands_ordering, int):
            operands_ordering = [operands_ordering]
        order = list(operands_ordering)
        return self._replace(paths=sorted(self.paths, key=lambda p: tuple(p.indices[i] for i in order)))

    def squeeze_modes(self, modes: Optional[str] = None) -> "SegmentedTensorProduct":
        """Drop the modes whose extent is 1 everywhere."""
        rm = {m for m, dd in self.get_dimensions_dict().items() if dd == {1}}
        if modes is not None:
            if not set(modes) <= rm:
                raise ValueError(f"modes {modes} cannot be squeezed.")
            rm &= set(modes)
        if not rm:
            return self

        def keep(shape, ss):
            return tuple(d for d, m in zip(shape, ss) if m not in rm)

        ops = [
            (SegmentedOperand([keep(s, ss) for s in ope], ndim=len([m for m in ss if m not in rm])),
             "".join(m for m in ss if m not in rm))
            for ope, ss in self.operands_and_subscripts
        ]
        cs = self.coefficient_subscripts
        paths = [Path(p.indices, np.reshape(p.coefficients, keep(p.coefficients.shape, cs))) for p in self.paths]
        return SegmentedTensorProduct(ops, "".join(m for m in cs if m not in rm), paths=paths)

    def split_mode(self, mode: str, size: int) -> "SegmentedTensorProduct":
        """Cut a leading mode into chunks of ``size``; each segment and path is subdivided accordingly."""
        if re.match(r"^[a-z]$", mode) is None:
            raise ValueError("expected a single lowercase letter.")
        if mode not in self.subscripts:
            return self
        for oid, (_, ss) in enumerate(self._ops):
            if mode in ss and not ss.startswith(mode):
                raise ValueError(f"mode {mode} is not the first mode in operand {oid} ({ss}).")
        if not all(d % size == 0 for d in self.get_dims(mode)):
            raise ValueError(f"mode {mode} is not divisible by {size}.")
        cs = self.coefficient_subscripts
        if mode in cs and not cs.startswith(mode):
            moved = mode + cs.replace(mode, "")
            perm = [cs.index(ch) for ch in moved]
            back = [moved.index(ch) for ch in cs]
            d = self._replace(
                paths=[Path(p.indices, np.transpose(p.coefficients, perm)) for p in self.paths],
                coefficient_subscripts=moved,
            ).split_mode(mode, size)
            return d._replace(
                paths=[Path(p.indices, np.transpose(p.coefficients, back)) for p in d.paths],
                coefficient_subscripts=cs,
            )

        ops, offsets_per_operand = [], []
        for ope, ss in self.operands_and_subscripts:
            if mode not in ss:
                ops.append((ope, ss))
                offsets_per_operand.append(None)
                continue
            segs, offs = [], []
            for s in ope:
                offs.append(len(segs))
                segs += [(size,) + s[1:]] * (s[0] // size)
            ops.append((SegmentedOperand(segs, ndim=ope.ndim), ss))
            offsets_per_operand.append(offs)
        paths = []
        for p in self.paths:
            n = self.get_path_dimensions_dict(p)[mode] // size
            for i in range(n):
                idx = [
                    s if offsets_per_operand[o] is None else offsets_per_operand[o][s] + i
                    for o, s in enumerate(p.indices)
                ]
                c = p.coefficients
                if cs.startswith(mode):
                    c = np.split(c, n, axis=0)[i]
                paths.append(Path(idx, c))
        return SegmentedTensorProduct(ops, cs, paths=paths)

    def normalize_paths_for_operand(self, operand: int) -> "SegmentedTensorProduct":
        """Scale coefficients so that each segment of ``operand`` has unit variance for unit-variance inputs.

        A path contributes ``mean(c^2) * prod(extent of every mode contracted away)`` to the
        variance of its output segment; all paths into a segment are divided by the square
        root of the segment's total.
        """
        operand = _canon(operand, self.num_operands, "operand")
        kept = set(self._ops[operand][1])
        all_ss = [ss for _, ss in self._ops] + [self.coefficient_subscripts]
        contracted = {m for i, ss in enumerate(all_ss) if i != operand for m in ss if m not in kept}
        var = [0.0] * self.operands[operand].num_segments
        for p in self.paths:
            dims = self.get_path_dimensions_dict(p)
            num = np.prod([d for m, d in dims.items() if m in contracted])
            var[p.indices[operand]] += np.mean(p.coefficients**2) * num
        paths = []
        for p in self.paths:
            v = var[p.indices[operand]]
            paths.append(Path(p.indices, p.coefficients / np.sqrt(v) if v > 0 else 0.0 * p.coefficients))
        return self._replace(paths=paths)

    def remove_zero_paths(self) -> "SegmentedTensorProduct":
        return self._replace(paths=[p for p in self.paths if not np.all(p.coefficients == 0)])

    def consolidate_paths(self) -> "SegmentedTensorProduct":
        """Merge paths with equal indices, drop zeros, sort by indices."""
        acc: dict = {}
        for p in self.paths:
            acc[p.indices] = acc[p.indices] + p.coefficients if p.indices in acc else np.array(p.coefficients)
        paths = [Path(i, c) for i, c in acc.items() if not np.all(c == 0)]
        return self._replace(paths=sorted(paths, key=lambda p: p.indices))

    def remove_empty_segments(self) -> "SegmentedTensorProduct":
        if all(d > 0 for dd in self.get_dimensions_dict().values() for d in dd):
            return self
        d = self
        for oid in range(self.num_operands):
            ope = d.operands[oid]
            keep = [i for i, s in enumerate(ope) if all(x > 0 for x in s)]
            drop = set(range(ope.num_segments)) - set(keep)
            new_index = {old: new for new, old in enumerate(keep)}
            ops = list(d.operands_and_subscripts)
            ops[oid] = (ope.with_segments([ope[i] for i in keep]), ops[oid][1])
            paths = [
                Path([new_index[s] if o == oid else s for o, s in enumerate(p.indices)], p.coefficients)
                for p in d.paths
                if p.indices[oid] not in drop
            ]
            d = d._replace(operands_and_subscripts=ops, paths=paths)
        return d

    def _check_scalar_coefficients_for(self, operands):
        if any(m in self.coefficient_subscripts for i in operands for m in self._ops[i][1]):
            raise NotImplementedError("flatten the coefficient modes first")

    def sort_indices_for_identical_operands(self, operands) -> "SegmentedTensorProduct":
        """For operands fed by the same buffer: sort each path's indices over them and merge duplicates."""
        operands = tuple(sorted(set(operands)))
        if len(operands) < 2:
            return self
        self._check_scalar_coefficients_for(operands)
        paths = []
        for p in self.paths:
            srt = sorted(p.indices[o] for o in operands)
            idx = list(p.indices)
            for o, s in zip(operands, srt):
                idx[o] = s
            paths.append(Path(idx, p.coefficients))
        return self._replace(paths=paths).consolidate_paths()

    def symmetrize_operands(self, operands) -> "SegmentedTensorProduct":
        """Spread every path evenly over all permutations of the given (identical) operands."""
        operands = tuple(sorted(set(operands)))
        if len(operands) < 2:
            return self
        self._check_scalar_coefficients_for(operands)
        d = self.sort_indices_for_identical_operands(operands)
        perms = list(itertools.permutations(range(len(operands))))
        paths = []
        for p in d.paths:
            for perm in perms:
                idx = list(p.indices)
                for i, o in enumerate(operands):
                    idx[o] = p.indices[operands[perm[i]]]
                paths.append(Path(idx, p.coefficients / len(perms)))
        return d._replace(paths=paths).consolidate_paths()

    def flatten_modes(self, modes, *, skip_zeros: bool = True) -> "SegmentedTensorProduct":
        """Remove leading modes by cutting every segment into one sub-segment per index of those modes.

        Sub-segment numbering: ``offset[segment] + ravel_multi_index(sub-index, removed shape)``.
        When every coefficient mode is removed, one scalar path is emitted per non-zero
        coefficient in row-major order (paths keep their relative order).
        """
        modes = "".join(sorted({m for m in modes if m in self.subscripts}))
        if not modes:
            return self
        pattern = re.compile(rf"^([{modes}]*)([^{modes}]*)$")
        ops, offs, rm_shapes, rm_modes = [], [], [], []
        for ope, ss in self.operands_and_subscripts:
            ma = pattern.match(ss)
            if ma is None:
                raise ValueError(f"expected modes {modes} to be at the beginning of the segment subscripts. Got {ss}.")
            rm, new_ss = ma.groups()
            n = len(rm)
            segs, o, shp, off = [], [], [], 0
            for s in ope:
                o.append(off)
                num = math.prod(s[:n])
                shp.append(s[:n])
                segs += [s[n:]] * num
                off += num
            ops.append((SegmentedOperand(segs, ndim=len(new_ss)), new_ss))
            offs.append(o)
            rm_shapes.append(shp)
            rm_modes.append(rm)

        def sub_path(old, sub: dict, c) -> Path:
            idx = []
            for sid, o, rm, shp in zip(old, offs, rm_modes, rm_shapes):
                k = int(np.ravel_multi_index(tuple(sub[m] for m in rm), shp[sid])) if rm else 0
                idx.append(o[sid] + k)
            return Path(idx, c)

        cs = self.coefficient_subscripts
        paths = []
        if skip_zeros and len(cs) > 0 and set(cs) <= set(modes):
            others = "".join(m for m in modes if m not in cs)
            for p in self.paths:
                dims = self.get_path_dimensions_dict(p)
                nz = np.nonzero(p.coefficients)
                vals = p.coefficients[nz]
                for oi in np.ndindex(tuple(dims[m] for m in others)):
                    d2 = dict(zip(others, oi))
                    for ci, c in zip(zip(*nz), vals):
                        paths.append(sub_path(p.indices, {**dict(zip(cs, ci)), **d2}, c))
        else:
            for p in self.paths:
                dims = self.get_path_dimensions_dict(p)
                for index in np.ndindex(tuple(dims[m] for m in modes)):
                    c = p.coefficients[tuple(index[modes.index(ch)] if ch in modes else slice(None) for ch in cs)]
                    if skip_zeros and np.all(c == 0):
                        continue
                    paths.append(sub_path(p.indices, dict(zip(modes, index)), c))
        return SegmentedTensorProduct(ops, "".join(ch for ch in cs if ch not in modes), paths=paths)

    def flatten_coefficient_modes(self, *, skip_zeros: bool = True) -> "SegmentedTensorProduct":
        return self.flatten_modes(self.coefficient_subscripts, skip_zeros=skip_zeros)

    def append_modes_to_all_operands(self, modes: str, dims: dict) -> "SegmentedTensorProduct":
        """Give every segment of every operand extra trailing modes of the given extents."""
        if any(ch in self.subscripts for ch in modes):
            raise ValueError(f"modes {modes} already present in {self.subscripts}")
        extra = tuple(dims[ch] for ch in modes)
        ops = [
            (SegmentedOperand([s + extra for s in ope], ndim=ope.ndim + len(modes)), ss + modes)
            for ope, ss in self.operands_and_subscripts
        ]
        return SegmentedTensorProduct(ops, self.coefficient_subscripts, paths=self.paths)

    def __mul__(self, factor: float) -> "SegmentedTensorProduct":
        return self._replace(paths=[Path(p.indices, p.coefficients * factor) for p in self.paths])

    __rmul__ = __mul__

    # ---------------------------------------------------------------- numpy evaluation
    def compute_last_operand(self, *inputs: np.ndarray, dtype=None) -> np.ndarray:
        """Reference numpy evaluation: inputs ``(..., operand_size)`` -> ``(..., last_operand_size)``."""
        if len(inputs) != self.num_operands - 1:
            raise ValueError(f"Expected {self.num_operands - 1} inputs, got {len(inputs)}.")
        for i, (ope, x) in enumerate(zip(self.operands, inputs)):
            if ope.size != x.shape[-1]:
                raise ValueError(f"Expected operand {i} to have size {ope.size}, got {x.shape[-1]}.")
        dtype = dtype or np.result_type(*inputs)
        batch = np.broadcast_shapes(*[x.shape[:-1] for x in inputs])
        sl = [o.segment_slices() for o in self.operands]
        ss = self.subscripts.operands
        formula = ",".join([self.coefficient_subscripts] + ["..." + s for s in ss[:-1]]) + "->..." + ss[-1]
        out = np.zeros(batch + (self.operands[-1].size,), dtype=dtype)
        for p in self.paths:
            segs = [
                np.reshape(inputs[o][..., sl[o][p.indices[o]]], inputs[o].shape[:-1] + self.operands[o][p.indices[o]])
                for o in range(self.num_operands - 1)
            ]
            r = np.einsum(formula, p.coefficients, *segs)
            out[..., sl[-1][p.indices[-1]]] += np.reshape(r, batch + (-1,))
        return out
