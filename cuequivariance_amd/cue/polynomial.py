"""Segmented polynomials: several segmented tensor products wired to input/output buffers.

Reference behaviour followed (``cuequivariance/cuequivariance``):

* ``segmented_polynomials/operation.py:50-316``            Operation (buffers, jvp, transpose)
* ``segmented_polynomials/segmented_polynomial.py:57-89``   operand sorting inside each operation, operations sorted by output
* ``segmented_polynomials/segmented_polynomial.py:1003-1133`` jvp / transpose / backward
* ``group_theory/equivariant_polynomial.py:28-622``         polynomial + per-operand representation metadata
"""

from __future__ import annotations

import itertools
from typing import Callable, Optional, Sequence

import numpy as np

from .irreps import IrrepsAndLayout
from .stp import SegmentedOperand, SegmentedTensorProduct

__all__ = ["Operation", "SegmentedPolynomial", "EquivariantPolynomial"]


class Operation:
    """Which buffer (inputs first, then outputs) feeds each operand of a tensor product."""

    __slots__ = ("buffers",)

    def __init__(self, buffers):
        if isinstance(buffers, Operation):
            buffers = buffers.buffers
        buffers = tuple(int(b) for b in buffers)
        assert len(buffers) > 0 and all(b >= 0 for b in buffers), buffers
        self.buffers = buffers

    def __repr__(self):
        return f"Operation({self.buffers})"

    def __hash__(self):
        return hash(self.buffers)

    def __eq__(self, o):
        return isinstance(o, Operation) and self.buffers == o.buffers

    def __lt__(self, o):
        return (len(self.buffers), self.buffers) < (len(o.buffers), o.buffers)

    def permute_operands(self, perm) -> "Operation":
        return Operation(tuple(self.buffers[p] for p in perm))

    def input_operands_buffers(self, num_inputs: int) -> list[tuple[int, int]]:
        return [(op, b) for op, b in enumerate(self.buffers) if b < num_inputs]

    def output_operand_buffer(self, num_inputs: int) -> tuple[int, int]:
        outs = [(op, b) for op, b in enumerate(self.buffers) if b >= num_inputs]
        if len(outs) != 1:
            raise ValueError(f"Operation must have exactly one output buffer. {self} num_inputs={num_inputs}")
        return outs[0]

    def input_buffers(self, num_inputs: int) -> list[int]:
        return [b for b in self.buffers if b < num_inputs]

    def output_buffer(self, num_inputs: int) -> int:
        return self.output_operand_buffer(num_inputs)[1]

    def jvp(self, has_tangent: Sequence[bool]) -> list["Operation"]:
        """One operation per operand slot whose buffer has a tangent.

        New buffer numbering: original inputs, then one tangent per ``True`` entry, then the outputs.
        """
        n_in = len(has_tangent)
        tangent_of, nxt = [], n_in
        for h in has_tangent:
            tangent_of.append(nxt if h else None)
            nxt += 1 if h else 0
        shift = nxt - n_in
        out_op, _ = self.output_operand_buffer(n_in)
        res = []
        for op, b in self.input_operands_buffers(n_in):
            if has_tangent[b]:
                nb = list(self.buffers)
                nb[op] = tangent_of[b]
                nb[out_op] += shift
                res.append(Operation(nb))
        return res

    def transpose(self, is_undefined_primal: Sequence[bool], has_cotangent: Sequence[bool]) -> Optional["Operation"]:
        """Swap the (single) undefined input with the output cotangent.

        New inputs: defined primals then cotangents; new outputs: the undefined primals.
        """
        n_in = len(is_undefined_primal)
        if not has_cotangent[self.output_buffer(n_in) - n_in]:
            return None
        undef = sum(1 for b in self.input_buffers(n_in) if is_undefined_primal[b])
        if undef > 1:
            raise ValueError(f"{self} has more than one undefined primal; it is not linear")
        if undef == 0:
            return None
        new_in, new_out_rel, k_in, k_out = [], [], 0, 0
        for u in is_undefined_primal:
            if u:
                new_in.append(None)
                new_out_rel.append(k_out)
                k_out += 1
            else:
                new_in.append(k_in)
                new_out_rel.append(None)
                k_in += 1
        cot = []
        for h in has_cotangent:
            cot.append(k_in if h else None)
            k_in += 1 if h else 0
        nb = []
        for b in self.buffers:
            if b < n_in:
                nb.append(k_in + new_out_rel[b] if is_undefined_primal[b] else new_in[b])
            else:
                nb.append(cot[b - n_in])
        return Operation(nb)

    def operands_with_identical_buffers(self) -> list[tuple[int, ...]]:
        groups: dict[int, list[int]] = {}
        for oid, b in enumerate(self.buffers):
            groups.setdefault(b, []).append(oid)
        return [tuple(g) for g in groups.values()]


class SegmentedPolynomial:
    """``outputs[k] = sum over operations writing k of stp(inputs...)``."""

    def __init__(self, inputs, outputs, operations):
        inputs, outputs = tuple(inputs), tuple(outputs)
        operands = inputs + outputs
        tmp = []
        for ope, stp in operations:
            ope = Operation(ope)
            assert isinstance(stp, SegmentedTensorProduct)
            assert len(ope.buffers) == stp.num_operands
            for b, o in zip(ope.buffers, stp.operands):
                assert o == operands[b], (b, o, operands[b])
            bid = ope.output_buffer(len(inputs))
            # Operands are put in buffer order (stable), so the output is always the last operand.
            perm = sorted(range(stp.num_operands), key=lambda i: ope.buffers[i])
            tmp.append((bid, ope.permute_operands(perm), stp.permute_operands(perm)))
        tmp.sort(key=lambda t: (t[0], t[1], t[2]))
        self.inputs = inputs
        self.outputs = outputs
        self.operations = tuple((ope, stp) for _, ope, stp in tmp)

    @classmethod
    def _from_default_operands(cls, inputs, outputs, operations):
        operands = list(inputs) + list(outputs)
        for ope, stp in operations:
            ope = Operation(ope)
            for b, o in zip(ope.buffers, stp.operands):
                operands[b] = o
        return cls(operands[: len(inputs)], operands[len(inputs):], operations)

    @classmethod
    def eval_last_operand(cls, stp: SegmentedTensorProduct) -> "SegmentedPolynomial":
        return cls(stp.operands[:-1], (stp.operands[-1],), ((Operation(range(stp.num_operands)), stp),))

    @classmethod
    def stack(cls, polys, stacked) -> "SegmentedPolynomial":
        """Stack polynomials: operands flagged in ``stacked`` are concatenated over ``polys`` (every tensor product keeps
        addressing its own slice), the others must be identical.  Operations with equal buffers are then fused
        (reference ``segmented_polynomial.py:167-232``)."""
        polys = list(polys)
        assert len(polys) > 0
        n_in, n_out = polys[0].num_inputs, polys[0].num_outputs
        assert all(p.num_inputs == n_in and p.num_outputs == n_out for p in polys)
        assert len(stacked) == n_in + n_out
        operands = []
        for bid in range(n_in + n_out):
            if stacked[bid]:
                parts = [p.operands[bid] for p in polys if p.operands[bid] is not None]
                operands.append(SegmentedOperand(sum([list(o.segments) for o in parts], []), ndim=parts[0].ndim))
            else:
                ope = polys[0].operands[bid]
                assert all(p.operands[bid] == ope for p in polys)
                operands.append(ope)
        ops = []
        for index, pol in enumerate(polys):
            for ope, stp in pol.operations:
                stp = stp.copy()
                for oid, b in enumerate(ope.buffers):
                    if stacked[b]:
                        for p in reversed(polys[:index]):
                            stp.insert_segments(oid, 0, p.operands[b].segments)
                        for p in polys[index + 1:]:
                            stp.insert_segments(oid, -1, p.operands[b].segments)
                ops.append((ope, stp))
        return cls(operands[:n_in], operands[n_in:], ops).consolidate()

    @classmethod
    def stack_tensor_products(cls, inputs, outputs, operations) -> "SegmentedPolynomial":
        """Operands given as ``None`` are the concatenation of that operand over all operations."""
        inputs, outputs = list(inputs), list(outputs)
        stacked = [o is None for o in inputs + outputs]
        n_in = len(inputs)
        polys = [cls._from_default_operands(inputs, outputs, [(o, s)]) for o, s in operations]
        operands = []
        for bid in range(len(stacked)):
            if stacked[bid]:
                parts = [p.operands[bid] for p in polys if p.operands[bid] is not None]
                operands.append(SegmentedOperand(sum([list(o.segments) for o in parts], []), ndim=parts[0].ndim))
            else:
                operands.append(polys[0].operands[bid])
        ops = []
        for index, pol in enumerate(polys):
            for ope, stp in pol.operations:
                stp = stp.copy()
                for oid, b in enumerate(ope.buffers):
                    if stacked[b]:
                        for p in reversed(polys[:index]):
                            stp.insert_segments(oid, 0, p.operands[b].segments)
                        for p in polys[index + 1:]:
                            stp.insert_segments(oid, -1, p.operands[b].segments)
                ops.append((ope, stp))
        return cls(operands[:n_in], operands[n_in:], ops)

    # ---------------------------------------------------------------- properties
    @property
    def operands(self):
        return self.inputs + self.outputs

    @property
    def num_inputs(self) -> int:
        return len(self.inputs)

    @property
    def num_outputs(self) -> int:
        return len(self.outputs)

    @property
    def num_operands(self) -> int:
        return self.num_inputs + self.num_outputs

    def __hash__(self):
        return hash((self.inputs, self.outputs, self.operations))

    def pack(self) -> str:
        """The polynomial as one line of text (operand shapes, and per operation its buffers and the tensor product's own
        ``to_base64``); ``unpack`` rebuilds an equal polynomial.  Traced graphs carry it in place of the object."""
        import json

        def shape(o):
            return [o.ndim, [list(seg) for seg in o.segments]]

        return json.dumps({"inputs": [shape(o) for o in self.inputs], "outputs": [shape(o) for o in self.outputs],
                           "operations": [[list(ope.buffers), stp.to_base64()] for ope, stp in self.operations]},
                          separators=(",", ":"))

    @classmethod
    def unpack(cls, text: str) -> "SegmentedPolynomial":
        import json

        data = json.loads(text)
        inputs = [SegmentedOperand(seg, ndim=ndim) for ndim, seg in data["inputs"]]
        outputs = [SegmentedOperand(seg, ndim=ndim) for ndim, seg in data["outputs"]]
        return cls(inputs, outputs, [(Operation(b), SegmentedTensorProduct.from_base64(t)) for b, t in data["operations"]])

    def __eq__(self, o):
        if not isinstance(o, SegmentedPolynomial):
            return NotImplemented
        return self.inputs == o.inputs and self.outputs == o.outputs and self.operations == o.operations

    def __repr__(self):
        names = "abcdefghijklmnopqrstuvwxyz"
        head = " ".join(f"{names[i]}=[{o.size}:{o.num_segments}]" for i, o in enumerate(self.inputs))
        head += " -> " + " ".join(
            f"{names[self.num_inputs + i].upper()}=[{o.size}:{o.num_segments}]" for i, o in enumerate(self.outputs)
        )
        lines = [head]
        for ope, stp in self.operations:
            letters = [names[b] if b < self.num_inputs else names[b].upper() for b in ope.buffers]
            lines.append(
                "  " + " ".join(f"{l}[{ss}]" for l, ss in zip(letters, stp.subscripts.operands))
                + f" [{stp.coefficient_subscripts}] num_paths={stp.num_paths}"
            )
        return "\n".join(lines)

    def __call__(self, *inputs: np.ndarray) -> list[np.ndarray]:
        """numpy evaluation (slow reference)."""
        shape = np.broadcast_shapes(*[x.shape[:-1] for x in inputs])
        dtype = np.result_type(*[x.dtype for x in inputs])
        outs = [np.zeros(shape + (o.size,), dtype=dtype) for o in self.outputs]
        for ope, stp in self.operations:
            oid, bid = ope.output_operand_buffer(self.num_inputs)
            outs[bid - self.num_inputs] += stp.move_operand_last(oid).compute_last_operand(
                *[inputs[b] for b in ope.input_buffers(self.num_inputs)], dtype=dtype
            )
        return outs

    def all_same_segment_shape(self) -> bool:
        return all(o.all_same_segment_shape() for o in self.operands)

    def used_inputs(self) -> list[bool]:
        return [any(i in ope.buffers for ope, _ in self.operations) for i in range(self.num_inputs)]

    def __mul__(self, f: float):
        return SegmentedPolynomial(self.inputs, self.outputs, [(o, s * f) for o, s in self.operations])

    __rmul__ = __mul__

    # ---------------------------------------------------------------- transforms
    def apply_fn(self, f: Callable) -> "SegmentedPolynomial":
        ops = [f(o, s) for o, s in self.operations]
        return SegmentedPolynomial._from_default_operands(self.inputs, self.outputs, [x for x in ops if x is not None])

    def flatten_modes(self, modes) -> "SegmentedPolynomial":
        return self.apply_fn(lambda o, s: (o, s.flatten_modes(modes)))

    def flatten_coefficient_modes(self) -> "SegmentedPolynomial":
        return self.apply_fn(lambda o, s: (o, s.flatten_coefficient_modes()))

    def squeeze_modes(self, modes: Optional[str] = None) -> "SegmentedPolynomial":
        ops = [(o, s.squeeze_modes(modes)) for o, s in self.operations]
        if modes is not None:
            ins, outs = self.inputs, self.outputs
        else:
            ins = tuple(o.squeeze() for o in self.inputs)
            outs = tuple(o.squeeze() for o in self.outputs)
        return SegmentedPolynomial._from_default_operands(ins, outs, ops)

    def split_mode(self, mode: str, size: int) -> "SegmentedPolynomial":
        return self.apply_fn(lambda o, s: (o, s.split_mode(mode, size)))

    def consolidate(self) -> "SegmentedPolynomial":
        """Fuse operations with the same buffers and operand structure, merge duplicate paths, drop empty ones."""
        groups: dict = {}
        order = []
        for ope, stp in self.operations:
            key = (ope, stp.operands_and_subscripts, stp.coefficient_subscripts)
            if key not in groups:
                groups[key] = []
                order.append(key)
            groups[key] += list(stp.paths)
        ops = []
        for key in order:
            ope, oas, cs = key
            stp = SegmentedTensorProduct(oas, cs, paths=groups[key]).remove_empty_segments().consolidate_paths()
            if stp.num_paths:
                ops.append((ope, stp))
        return SegmentedPolynomial._from_default_operands(self.inputs, self.outputs, ops).squeeze_modes()

    def symmetrize_for_identical_operands(self) -> "SegmentedPolynomial":
        ops = []
        for ope, stp in self.operations:
            for grp in ope.operands_with_identical_buffers():
                stp = stp.symmetrize_operands(grp)
            ops.append((ope, stp.sort_paths()))
        return SegmentedPolynomial(self.inputs, self.outputs, ops)

    def unsymmetrize_for_identical_operands(self) -> "SegmentedPolynomial":
        def f(ope, stp):
            for grp in ope.operands_with_identical_buffers():
                stp = stp.sort_indices_for_identical_operands(grp)
            return ope, stp.sort_paths()

        return self.apply_fn(f)

    # ---------------------------------------------------------------- differentiation
    def jvp(self, has_tangent: Sequence[bool]):
        """Polynomial of the directional derivative; inputs = originals + tangents (for ``True`` entries).

        Operations that differ only by which of several identical operand slots carries the
        tangent are merged into one with an integer multiplicity when the (symmetrised)
        tensor product is invariant under exchanging those slots.
        """
        assert len(has_tangent) == self.num_inputs
        sym = self.symmetrize_for_identical_operands()
        ops = []
        for ope, stp in sym.operations:
            jv = ope.jvp(has_tangent)
            seen: dict = {}
            for j in jv:
                # operations equal up to a permutation among slots bound to one original buffer
                key = tuple(sorted(zip(_slot_classes(ope), j.buffers)))
                seen.setdefault(key, []).append(j)
            for group in seen.values():
                ops.append((sorted(group)[0], len(group) * stp))

        def mapping(x, into_grad=None):
            ins, outs = list(x[0]), list(x[1])
            g = into_grad if callable(into_grad) else (lambda v: v)
            return ins + [g(v) for h, v in zip(has_tangent, ins) if h], [g(v) for v in outs]

        return SegmentedPolynomial(*mapping((self.inputs, self.outputs)), ops), mapping

    def transpose(self, is_undefined_primal: Sequence[bool], has_cotangent: Sequence[bool]):
        assert len(is_undefined_primal) == self.num_inputs and len(has_cotangent) == self.num_outputs
        ops = []
        for ope, stp in self.operations:
            t = ope.transpose(is_undefined_primal, has_cotangent)
            if t is not None:
                ops.append((t, stp))

        def mapping(x):
            ins, outs = list(x[0]), list(x[1])
            new_in = [v for u, v in zip(is_undefined_primal, ins) if not u] + [
                v for h, v in zip(has_cotangent, outs) if h
            ]
            return new_in, [v for u, v in zip(is_undefined_primal, ins) if u]

        return SegmentedPolynomial(*mapping((self.inputs, self.outputs)), ops), mapping

    def backward(self, requires_gradient: Sequence[bool], has_cotangent: Sequence[bool]):
        """Polynomial mapping ``(inputs, output cotangents) -> input gradients``."""
        p, m1 = self.jvp(requires_gradient)
        p, m2 = p.transpose([False] * self.num_inputs + [True] * sum(requires_gradient), has_cotangent)
        return p, (lambda x, into_grad=None: m2(m1(x, into_grad)))


def _slot_classes(ope: Operation) -> list[int]:
    """Label each operand slot by the original buffer it reads, so symmetric slots share a label."""
    return list(ope.buffers)


class EquivariantPolynomial:
    """A segmented polynomial whose operands are annotated with irreps and layouts."""

    def __init__(self, inputs, outputs, polynomial: SegmentedPolynomial):
        self.inputs = tuple(inputs)
        self.outputs = tuple(outputs)
        self.polynomial = polynomial
        assert len(self.inputs) == polynomial.num_inputs and len(self.outputs) == polynomial.num_outputs
        for rep, ope in zip(self.inputs + self.outputs, polynomial.operands):
            assert rep.dim == ope.size, f"{rep.dim} != {ope.size} for {rep}"

    @property
    def operands(self):
        return self.inputs + self.outputs

    @property
    def num_inputs(self):
        return len(self.inputs)

    @property
    def num_outputs(self):
        return len(self.outputs)

    def __repr__(self):
        return " ".join(map(repr, self.inputs)) + " -> " + " ".join(map(repr, self.outputs)) + "\n" + repr(self.polynomial)

    def _with(self, poly):
        return EquivariantPolynomial(self.inputs, self.outputs, poly)

    def flatten_coefficient_modes(self):
        return self._with(self.polynomial.flatten_coefficient_modes())

    def flatten_modes(self, modes):
        return self._with(self.polynomial.flatten_modes(modes))

    def squeeze_modes(self, modes=None):
        return self._with(self.polynomial.squeeze_modes(modes))

    def split_mode(self, mode, size):
        return self._with(self.polynomial.split_mode(mode, size))

    def all_same_segment_shape(self) -> bool:
        return self.polynomial.all_same_segment_shape()

    def __call__(self, *inputs):
        return self.polynomial(*inputs)
