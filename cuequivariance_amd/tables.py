"""Flat uniform-1d path tables (torch-free): construction from a polynomial, transposition, hashing.

The table layout is the one the reference builds at
``cuequivariance_torch/cuequivariance_torch/primitives/segmented_polynomial_uniform_1d.py:188-218``.
"""

from __future__ import annotations

import struct
from dataclasses import dataclass, field
from itertools import accumulate
from typing import Optional, Sequence

_MASK64 = (1 << 64) - 1


@dataclass(frozen=True)
class U1dTables:
    operand_extent: int
    num_inputs: int
    num_outputs: int
    buffer_dim: tuple
    buffer_num_segments: tuple
    dtypes: tuple
    num_operands: tuple
    operations: tuple
    num_paths: tuple
    path_indices_start: tuple
    path_coefficients_start: tuple
    path_indices: tuple
    path_coefficients: tuple
    # Optional layout of the rows of channel-carrying buffers: per buffer either () - segment s, channel u at
    # s * extent + u ("ir_mul": channels contiguous) - or the sizes (d_0, d_1, ...) of groups of consecutive segments whose
    # rows are stored channel-major inside the group ("mul_ir": segment c of group g, channel u at
    # extent * (d_0 + ... + d_{g-1}) + u * d_g + c).  () for the whole field: every buffer in the default layout.
    layouts: tuple = ()

    @classmethod
    def make(cls, operand_extent, num_inputs, num_outputs, buffer_dim, buffer_num_segments, dtypes, num_operands,
             operations, num_paths, path_indices_start, path_coefficients_start, path_indices, path_coefficients):
        t = cls(
            int(operand_extent), int(num_inputs), int(num_outputs),
            tuple(int(x) for x in buffer_dim), tuple(int(x) for x in buffer_num_segments),
            tuple(int(x) for x in dtypes), tuple(int(x) for x in num_operands), tuple(int(x) for x in operations),
            tuple(int(x) for x in num_paths), tuple(int(x) for x in path_indices_start),
            tuple(int(x) for x in path_coefficients_start), tuple(int(x) for x in path_indices),
            tuple(float(x) for x in path_coefficients),
        )
        nbuf = t.num_inputs + t.num_outputs
        if len(t.buffer_dim) != nbuf or len(t.buffer_num_segments) != nbuf or len(t.dtypes) != nbuf:
            raise ValueError("uniform_1d: per-buffer lists must have num_inputs + num_outputs entries")
        if not (len(t.num_operands) == len(t.num_paths) == len(t.path_indices_start) == len(t.path_coefficients_start)):
            raise ValueError("uniform_1d: per-operation lists have inconsistent lengths")
        if sum(t.num_operands) != len(t.operations):
            raise ValueError("uniform_1d: `operations` does not match `num_operands`")
        return t

    @classmethod
    def from_polynomial(cls, polynomial, output_dtype_map: Optional[Sequence[int]] = None) -> "U1dTables":
        """``polynomial`` must already be flattened to scalar coefficients with at most one (uniform) mode."""
        extent = None
        for o in polynomial.operands:
            if o.ndim not in (0, 1):
                raise ValueError("uniform_1d: only 0-d or 1-d operands are supported")
            if not o.all_same_segment_shape():
                raise ValueError("uniform_1d: all segments of an operand must have the same shape")
            if o.ndim == 1 and len(o.segments) > 0:
                (e,) = o.segment_shape
                if extent is None:
                    extent = e
                elif extent != e:
                    raise ValueError("uniform_1d: all 1-d operands must share the same segment extent")
        extent = 1 if extent is None else extent
        ops = polynomial.operations
        for ope, stp in ops:
            if stp.num_operands != len(ope.buffers) or stp.coefficient_subscripts != "":
                raise ValueError("uniform_1d: coefficients must be scalar")
        nin, nout = polynomial.num_inputs, polynomial.num_outputs
        default_map = [0 if nin >= 1 else -1] * nout
        return cls.make(
            extent, nin, nout,
            [o.ndim for o in polynomial.operands],
            [len(o.segments) for o in polynomial.operands],
            list(range(nin)) + (default_map if output_dtype_map is None else list(output_dtype_map)),
            [len(o.buffers) for o, _ in ops],
            [b for o, _ in ops for b in o.buffers],
            [s.num_paths for _, s in ops],
            [0] + list(accumulate(s.num_paths * s.num_operands for _, s in ops))[:-1],
            [0] + list(accumulate(s.num_paths for _, s in ops))[:-1],
            [i for _, s in ops for p in s.paths for i in p.indices],
            [float(p.coefficients) for _, s in ops for p in s.paths],
        )

    def width(self, b: int) -> int:
        return self.buffer_num_segments[b] * (self.operand_extent if self.buffer_dim[b] else 1)

    def layout(self, b: int) -> tuple:
        return self.layouts[b] if self.layouts else ()

    def with_layouts(self, groups: dict) -> "U1dTables":
        """The same tables with the rows of the buffers in ``groups`` ({buffer: group sizes}) stored group by group,
        channel-major inside a group (the ``mul_ir`` layout of an irreps operand: one group per ``(mul, ir)`` block)."""
        from dataclasses import replace

        nbuf = self.num_inputs + self.num_outputs
        lay = [tuple(self.layout(b)) for b in range(nbuf)]
        for b, dims in groups.items():
            dims = tuple(int(d) for d in dims)
            if not self.buffer_dim[b] or sum(dims) != self.buffer_num_segments[b] or any(d < 1 for d in dims):
                raise ValueError(f"uniform_1d: groups {dims} do not partition the {self.buffer_num_segments[b]} channel segments of buffer {b}")
            lay[b] = () if all(d == 1 for d in dims) else dims  # groups of one segment are the default layout
        return replace(self, layouts=tuple(lay) if any(lay) else ())

    def segment_addressing(self, b: int):
        """(base offset, channel stride) of every segment of buffer ``b`` under its layout."""
        E = self.operand_extent if self.buffer_dim[b] else 1
        dims = self.layout(b)
        if not dims:
            return [(seg * E, 1) for seg in range(self.buffer_num_segments[b])]
        out, off = [], 0
        for d in dims:
            out += [(off + c, d) for c in range(d)]
            off += d * E
        return out

    def operation(self, o: int):
        """(buffers, [(indices..., coefficient)]) of operation ``o``."""
        off = sum(self.num_operands[:o])
        nop = self.num_operands[o]
        bufs = self.operations[off: off + nop]
        pi0, pc0 = self.path_indices_start[o], self.path_coefficients_start[o]
        paths = [
            (self.path_indices[pi0 + p * nop: pi0 + (p + 1) * nop], self.path_coefficients[pc0 + p])
            for p in range(self.num_paths[o])
        ]
        return bufs, paths

    def backward(self, needs_grad: Sequence[bool]) -> "U1dTables":
        """Tables computing the gradients of the inputs flagged in ``needs_grad``.

        Buffers of the result: the original inputs, one cotangent per original output, then one
        gradient per flagged input.  For every operation and every operand slot bound to a flagged
        input, an operation with the same path table is emitted in which that slot becomes the
        output and the original output slot reads the cotangent (transposition relabels buffers and
        leaves the path table untouched).
        """
        nin, nout = self.num_inputs, self.num_outputs
        grad_buf, k = {}, nin + nout
        for i, g in enumerate(needs_grad):
            if g:
                grad_buf[i] = k
                k += 1
        buf_dim = list(self.buffer_dim) + [self.buffer_dim[i] for i in grad_buf]
        buf_nseg = list(self.buffer_num_segments) + [self.buffer_num_segments[i] for i in grad_buf]
        dtypes = list(range(nin + nout)) + [i for i in grad_buf]
        num_operands, operations, num_paths, pis, pcs = [], [], [], [], []
        off = 0
        for o, nop in enumerate(self.num_operands):
            bufs = self.operations[off: off + nop]
            off += nop
            out_pos = [s for s, b in enumerate(bufs) if b >= nin]
            assert len(out_pos) == 1
            out_pos = out_pos[0]
            for s, b in enumerate(bufs):
                if s == out_pos or not needs_grad[b]:
                    continue
                nb = list(bufs)
                nb[s] = grad_buf[b]  # nb[out_pos] keeps its id: the cotangent of output j is buffer nin + j
                num_operands.append(nop)
                operations += nb
                num_paths.append(self.num_paths[o])
                pis.append(self.path_indices_start[o])
                pcs.append(self.path_coefficients_start[o])
        out = U1dTables.make(
            self.operand_extent, nin + nout, len(grad_buf), buf_dim, buf_nseg, dtypes, num_operands, operations,
            num_paths, pis, pcs, self.path_indices, self.path_coefficients,
        )
        if self.layouts:  # cotangents keep the layout of their output, gradients that of their input
            lay = {b: self.layout(b) for b in range(nin + nout) if self.layout(b)}
            lay.update({g: self.layout(i) for i, g in grad_buf.items() if self.layout(i)})
            out = out.with_layouts(lay)
        return out

    def pack(self) -> str:
        """The tables as one line of text (two base64 fields of deflated bytes: the integers as little-endian int64, the
        coefficients as float64): what a traced graph carries in place of the object, so that a saved graph can be loaded
        where the object does not exist.  ``unpack`` inverts it exactly."""
        import base64
        import zlib

        nbuf = self.num_inputs + self.num_outputs
        lay = []
        for b in range(nbuf if self.layouts else 0):
            lay += [len(self.layouts[b]), *self.layouts[b]]
        ints = [self.operand_extent, self.num_inputs, self.num_outputs, len(self.num_operands), len(self.operations),
                len(self.path_indices), len(self.path_coefficients), len(lay),
                *self.buffer_dim, *self.buffer_num_segments, *self.dtypes, *self.num_operands, *self.operations, *self.num_paths,
                *self.path_indices_start, *self.path_coefficients_start, *self.path_indices, *lay]
        a = base64.b64encode(zlib.compress(struct.pack(f"<{len(ints)}q", *ints), 6)).decode("ascii")
        c = base64.b64encode(zlib.compress(struct.pack(f"<{len(self.path_coefficients)}d", *self.path_coefficients), 6)).decode("ascii")
        return a + ":" + c

    @classmethod
    def unpack(cls, text: str) -> "U1dTables":
        import base64
        import zlib

        a, c = text.split(":")
        raw = zlib.decompress(base64.b64decode(a))
        ints = list(struct.unpack(f"<{len(raw) // 8}q", raw))
        extent, nin, nout, nops, noperations, nidx, ncoef, nlay = ints[:8]
        pos = [8]

        def take(n):
            out = ints[pos[0]: pos[0] + n]
            pos[0] += n
            return out

        nbuf = nin + nout
        buffer_dim, nseg, dtypes = take(nbuf), take(nbuf), take(nbuf)
        num_operands, operations, num_paths, pis, pcs = take(nops), take(noperations), take(nops), take(nops), take(nops)
        path_indices, lay = take(nidx), take(nlay)
        if pos[0] != len(ints):
            raise ValueError("uniform_1d: packed tables of unexpected length")
        raw = zlib.decompress(base64.b64decode(c))
        coefficients = struct.unpack(f"<{ncoef}d", raw)
        t = cls.make(extent, nin, nout, buffer_dim, nseg, dtypes, num_operands, operations, num_paths, pis, pcs, path_indices, coefficients)
        if lay:
            groups, k = {}, 0
            for b in range(nbuf):
                n = lay[k]
                if n:
                    groups[b] = lay[k + 1: k + 1 + n]
                k += 1 + n
            t = t.with_layouts(groups)
        return t

    def content_hash(self, math_code: int) -> int:
        """FNV-1a 64 over the table contents; equals ``cueq::hash_u1d_desc`` of the C library."""
        words = [math_code, self.operand_extent, self.num_inputs, self.num_outputs, *self.buffer_dim,
                 *self.buffer_num_segments, len(self.num_operands)]
        off = 0
        for o, nop in enumerate(self.num_operands):
            words.append(nop)
            words += list(self.operations[off: off + nop])
            off += nop
            words.append(self.num_paths[o])
            pi0, pc0 = self.path_indices_start[o], self.path_coefficients_start[o]
            words += list(self.path_indices[pi0: pi0 + self.num_paths[o] * nop])
            for p in range(self.num_paths[o]):
                words.append(struct.unpack("<Q", struct.pack("<d", self.path_coefficients[pc0 + p]))[0])
        if self.layouts:  # (tables without layouts hash as they always did)
            words.append(0x6C61796F757473)
            for lay in self.layouts:
                words.append(len(lay))
                words += list(lay)
        h = 1469598103934665603
        for w in words:
            w &= _MASK64
            for i in range(8):
                h ^= (w >> (8 * i)) & 0xFF
                h = (h * 1099511628211) & _MASK64
        return h
